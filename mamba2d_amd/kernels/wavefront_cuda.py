"""Import-path twin of the reference's ``models/kernels/wavefront_cuda.py``: a model file
that does ``from .kernels.wavefront_cuda import wavefront_scan_cuda`` (models/mamba2d.py:10)
finds the same names here."""
from ..wavefront import (fused_backward_math, proj_params, scan_bwd_op, scan_fwd_op, wavefront_scan_cuda,  # noqa: F401
                         wf_bwd_op, wf_cuda_fn_fr, wf_cuda_fn_pr, wf_fwd_op)
