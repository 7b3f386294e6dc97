"""jax.numpy of the model: numpy itself, with float16 standing in for bfloat16 (two bytes, which is all
the binding's shape / dtype bookkeeping looks at)."""
from numpy import *  # noqa: F401,F403
from numpy import float16 as bfloat16  # noqa: F401
