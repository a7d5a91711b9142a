"""MI355X drop-in for the reference's `attention_variants` package.

Same module names, function names, positional parameters and result layouts as the reference's eager definitions
(attention_variants/*.py); where callers of the reference write `torch.compile(fn)(q, k, v, ...)`, callers of this
package call `fn(q, k, v, ...)` and get one fused HIP kernel launch on the current stream.
Inputs must be bfloat16 (or float16) tensors on a GPU; anything else raises (there is no eager fallback).
"""
from .vanilla import attention_pytorch, attention_pytorch_nogqa  # noqa: F401
from .causal import attention_pytorch_causal  # noqa: F401
from .alibi import alibi_bias, attention_pytorch_alibi, generate_alibi_bias_pytorch  # noqa: F401
from .softcap import attention_softcapped, generate_tanh_softcap  # noqa: F401
from .sliding_window import attention_pytorch_sliding_window, get_sliding_mask  # noqa: F401
from .prefix_lm import attention_pytorch_prefix_lm, get_prefix_lm_mask  # noqa: F401
from .document_mask import DocumentMaskWorkspace, attention_pytorch_document_mask, create_document_id  # noqa: F401
from .diff_attn import diffattn  # noqa: F401
from .evoformer import attention_reference  # noqa: F401
from .ipa import invariant_point_attention  # noqa: F401
from ._common import honor_dropout  # noqa: F401
