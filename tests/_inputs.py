"""The seeded synthetic inputs of the tests live in the package (flash_colreduce_amd/workloads.py), where
the benchmark and the smoke test take them from as well."""
from flash_colreduce_amd.workloads import *  # noqa: F401,F403
