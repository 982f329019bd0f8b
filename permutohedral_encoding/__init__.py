"""Drop-in import name: ``import permutohedral_encoding`` resolves to the MI355X implementation."""
from permutohedral_encoding_amd import *  # noqa: F401,F403
from permutohedral_encoding_amd import __all__  # noqa: F401
