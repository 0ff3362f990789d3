"""dmf_amd -- MI355X-native forward-mode (JVP) attention for Decoupled MeanFlow.

The public surface mirrors the reference's attention path:

* ``flash_attn_func(q, k, v, softmax_scale=None)`` -- dual in / dual out
  (reference: models/flash_attention_2_jvp.py:294-319),
* ``FlashAttnFunc`` -- the ``torch.autograd.Function`` with ``forward`` /
  ``setup_context`` / ``backward`` / ``jvp`` (reference: :177-282),
* ``attn_op(q, k, v, op)`` with the extra value ``op="hip"``
  (reference: models/layers.py:86-115).

All device work is done by hand-written gfx950 kernels reached through the
C ABI in ``include/dmf_attn.h`` (``dmf_amd/libdmf_attn.so``); there is no
fallback path: if the library is missing, calls raise.
"""
from .flash_attention_hip_jvp import (FlashAttnFunc, FlashAttnQKVPackedFunc, QKNormAttnQKVPackedFunc, flash_attn_func,  # noqa: F401
                                      flash_attn_qknorm_qkvpacked_func, flash_attn_qkvpacked_func)
from .layers import attn_op, ATTN_FUNCS  # noqa: F401
