"""Client loops and model definitions the launcher starts as threads."""
