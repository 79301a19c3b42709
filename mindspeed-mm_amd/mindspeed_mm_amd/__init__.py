"""MI355X-native Gated DeltaNet operator path: chunked rule (fwd+bwd), fused recurrent decode and the causal short
conv1d, plus the steps on either side of them in the layer (gate recipe, gated RMSNorm), behind the reference's Python
entry-point signatures.  The kernels are hand-written HIP for gfx950 in lib/libgdn_mi355x.so (sources under ../csrc);
there is no other execution path."""
from .ops import (GdnDecodeCache, GdnOps, RMSNormGated, ShortConvolution, causal_conv1d, causal_conv1d_update, chunk_gated_delta_rule,
                  chunk_gated_delta_rule_norm, chunk_gated_delta_rule_qkv, chunk_kda, decode_step, fused_recurrent_gated_delta_rule,
                  fused_recurrent_gated_delta_rule_qkv, gdn_gates, rms_norm_gated)

from . import library   # registers torch.ops.mindspeed_mm_amd.* (the same entry points as torch.library operators)

__all__ = ["GdnDecodeCache", "GdnOps", "RMSNormGated", "ShortConvolution", "causal_conv1d", "causal_conv1d_update",
           "chunk_gated_delta_rule", "chunk_gated_delta_rule_norm", "chunk_gated_delta_rule_qkv", "chunk_kda", "decode_step", "fused_recurrent_gated_delta_rule",
           "fused_recurrent_gated_delta_rule_qkv", "gdn_gates", "library", "rms_norm_gated"]
