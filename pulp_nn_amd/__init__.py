"""PULP-NN's int8 kernel set on MI355X: Python front end of the C-ABI libraries.

    from pulp_nn_amd import PulpNN
    nn = PulpNN(32)                       # or 64: width of k / lambda
    nn.set_batch(256)
    nn.pulp_nn_pointwise_HoWo_parallel(x, None, bias, y, w, None, None, mult, shift, ...)

Method names and argument lists are those of the reference's pulp_nn_kernels.h;
pointer arguments take torch tensors on the GPU (or raw device addresses).
There is no CPU fallback: loading fails if the HIP libraries have not been built
(python -m pulp_nn_amd.build).
"""
from .api import PulpNN, PulpNNError, lib_path  # noqa: F401
