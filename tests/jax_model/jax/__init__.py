"""A minimal numpy-backed MODEL of the part of the JAX API that olmax_amd/jax_ffi.py uses.

Test infrastructure only (this image has no JAX): it lets tests/test_ffi_binding.py run the binding's
wrappers and their custom_vjp rules on the CPU and record every ``jax.ffi.ffi_call`` they make, which
the test then compares with the handler bindings of olmax_amd/ffi/olmax_ffi.cc (operand count, result
count, attribute names and types).  Custom calls return zero-filled arrays of the requested shapes;
nothing is computed and nothing here is part of the product."""
from . import ffi, numpy, tree, tree_util  # noqa: F401


class ShapeDtypeStruct:
    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(shape), dtype


class custom_vjp:
    """jax.custom_vjp: calling it runs the primal function; the rules given to defvjp are kept so that a
    test can run them the way JAX does (fwd with all arguments in order; bwd with the non-differentiable
    arguments first, then the residuals, then the cotangent)."""

    def __init__(self, fun, nondiff_argnums=()):
        self.fun, self.nondiff_argnums = fun, tuple(nondiff_argnums)
        self.fwd = self.bwd = None

    def defvjp(self, fwd, bwd):
        self.fwd, self.bwd = fwd, bwd

    def _check_static(self, args):
        # JAX refuses array values (tracers, under jit) in nondiff_argnums: they must be static Python values
        import numpy as np
        for i in self.nondiff_argnums:
            assert not isinstance(args[i], np.ndarray), f"argument {i} is an array but is listed in nondiff_argnums"

    def __call__(self, *args):
        self._check_static(args)
        return self.fun(*args)

    def run_vjp(self, *args, cotangent=None):
        """-> (primal output, gradients of the differentiable arguments), through fwd and bwd."""
        self._check_static(args)
        out, res = self.fwd(*args)
        nondiff = [args[i] for i in self.nondiff_argnums]
        ct = cotangent if cotangent is not None else tree.map(lambda o: numpy.ones_like(o), out)
        grads = self.bwd(*nondiff, res, ct)
        assert len(grads) == len(args) - len(nondiff), "bwd must return one cotangent per differentiable argument"
        return out, grads


def jit(fun, donate_argnums=(), **_):
    return fun
