"""optax of the model: the one type the binding returns."""
from collections import namedtuple

GradientTransformation = namedtuple("GradientTransformation", ["init", "update"])
