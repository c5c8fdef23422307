"""brainpylib_amd: brainpylib's event-driven sparse operators for one AMD Instinct MI355X.

Same operator names, keyword arguments and semantics as ``brainpylib`` for the path that matters
in a spiking-network step (``event_csr_matvec``, ``csr_matvec``, the jitconn family); the
operators take and return ``torch`` tensors on the GPU and run hand-written gfx950 kernels through
the XLA custom-call ABI exported by ``lib/libbrainpylib_amd.so``.  There is no CPU fallback.
"""
__version__ = "0.1.0"

from ._lib import GPUOperatorNotFound
from .event_ops import event_csr_matvec, event_csr_matvec_batching, event_info
from .sparse_ops import check_csr, coo_to_csr, csr_matvec, csr_to_coo, csr_to_dense, cusparse_csr_matvec
from . import compat, jitconn_ops
from .compat import coo_atomic_prod, coo_atomic_sum, coo_event_sum, csr_event_prod, csr_event_sum
from .jitconn_ops import *  # noqa: F401,F403

__all__ = ["event_csr_matvec", "event_csr_matvec_batching", "event_info", "csr_matvec", "cusparse_csr_matvec", "csr_to_coo",
           "coo_to_csr", "csr_to_dense", "check_csr", "csr_event_sum", "coo_event_sum", "coo_atomic_sum", "csr_event_prod",
           "coo_atomic_prod", "compat",
           "GPUOperatorNotFound",
           "jitconn_ops"] + jitconn_ops.__all__
