"""MI355X-native (gfx950) dense-contraction kernels behind DNNKernels' kernel entry points.

``juliavision_amd.kernels`` mirrors the reference's ``matmul!`` / ``batchedmatmul!`` /
``sdpa`` / ``convolution!`` / ``layernorm!`` over the C ABI of ``libmi355dnn.so``
(declared in ``include/mi355dnn.h``).  Importing this package loads nothing; the
shared object is opened on first use and its absence is an error, never a fallback.
``juliavision_amd.decode`` holds the device-resident KV cache and the replayable
decoder-layer step, ``juliavision_amd.encoder`` the encoder block and a ViT-style
encoder composed from the same entry points, ``juliavision_amd.graph`` a loader/executor
for exported op graphs in the reference's JSON schema, ``juliavision_amd.safetensors``
the weight-file reader.
"""
from . import _lib  # noqa: F401
from .kernels import (Ctx, Decline, DeclineError, DeviceCaps, MI355X, Workspace, act_, add_, batchedmatmul_, caps, clamp_, conv_plan,
                      convolution_, convolution_nhwc_, convolution_tokens_, convolutiontranspose_, convsize, convtranspose_plan, convtransposesize, layernorm_, ln_matmul_, lnfold_matmul_, lnfold_prepare, matmul_rowstats_, rowstats_, rowstats_new, LnFoldedLinear, matmul_, matmul_heads_, matmul_ln_, mmplan, relayout_weight, scale_, sdpa, sdpa_append, sdpaplan, softmax_, transposeLE_)

__all__ = ["Ctx", "Decline", "DeclineError", "DeviceCaps", "MI355X", "Workspace", "act_", "add_", "batchedmatmul_", "caps", "clamp_",
           "conv_plan", "convolution_", "convolution_nhwc_", "convolution_tokens_", "convolutiontranspose_", "convsize", "convtranspose_plan", "convtransposesize", "layernorm_", "ln_matmul_", "lnfold_matmul_", "lnfold_prepare", "matmul_rowstats_", "rowstats_", "rowstats_new", "LnFoldedLinear", "matmul_", "matmul_heads_", "matmul_ln_", "mmplan", "relayout_weight", "scale_", "sdpa", "sdpa_append", "sdpaplan", "softmax_", "transposeLE_"]
