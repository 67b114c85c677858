"""Building the scheduler's profile files on gfx950."""
