"""Seeded synthetic inputs of the tests: the generators live in eisen_amd.synth (bench.py uses them too)."""
from eisen_amd.synth import *  # noqa: F401,F403
