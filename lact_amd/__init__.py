"""lact_amd: MI355X-native large-chunk SwiGLU fast-weight TTT operation (LaCT).

The package mirrors the reference's call signatures for this one path:
  lact_amd.ttt_operation  <- lact_llm/lact_model/ttt_operation.py
  lact_amd.minimal        <- minimal_implementations/*.py (operations)
  lact_amd.nvs            <- lact_nvs/lact_ttt.py (operation)
  lact_amd.ar_video       <- lact_ar_video/minVid/models/blocks/ar_lact_swa_repeat{,_sp}.py (operations)
  lact_amd.layers         <- minimal_implementations/bidirectional_lact_layer.py, causal_lact_with_sliding_window_attn.py
                             (the two layer classes around the operation)
All arithmetic runs in lib/liblact_hip.so (built from csrc/ with hipcc for gfx950)."""
from .ops import NS5_COEFFS, NS_CLASSIC, Program, block_causal_steps, check_async_error, run_program  # noqa: F401
from .ttt_operation import (block_causal_lact_swiglu, l2_norm, prenorm_block_causal_lact_swiglu,  # noqa: F401
                            postnorm_block_causal_lact_swiglu_fused_kernel_triton,
                            prenorm_block_causal_lact_swiglu_fused_kernel_triton,
                            silu_backprop, zeropower_via_newtonschulz5)
from .minimal import bidirectional_lact_swiglu, inv_softplus  # noqa: F401
from .nvs import TTTOperator, fast_weight_swish_glu_weight_norm_mini_batch_apply  # noqa: F401
from .layers import (BidirectionalLaCTSwiGLU, CausalLaCTSwiGLUWithSlidingWindowAttn, FastWeightGluMLPMultihead,  # noqa: F401
                     sliding_window_attention)
