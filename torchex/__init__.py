"""Drop-in spelling: ``from torchex import scatter_sum, scatter_max, scatter_mean,
TorchTimer, ScatterData`` (the import line of the reference's
``test/test_scatter.py:4``) resolves to the MI355X implementation."""
from torchex_amd import *  # noqa: F401,F403
from torchex_amd import __all__  # noqa: F401
