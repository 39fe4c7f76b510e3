"""Seeded synthetic inputs shared by the parity tests."""
from recsdk_amd.synth import splitmix64, zipf_keys, zipf_ranks  # noqa: F401
