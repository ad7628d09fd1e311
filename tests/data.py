"""The seeded synthetic inputs live in the package (vq_amd/synth.py: bench.py and smoke() use
them too); the tests import them under this name."""
from vq_amd.synth import F, gaussian_mixture, index_streams, uniform, unit_rows  # noqa: F401
