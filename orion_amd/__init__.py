"""orion_amd: an MI355X-native implementation of the Orion GPU-sharing hot path.

Interception -> per-client hand-off queues -> the Orion policy poll loop ->
dispatch on CU-masked HIP streams, behind the reference's own job API
(reference: benchmarking/launch_jobs.py, src/scheduler_frontend.py).
"""

__version__ = "0.1.0"
