"""kvhip: MI355X (gfx950) KV-cache hot path behind the reference's KVCache surface."""
from ._lib import KVHipError, LIB_PATH, SIGNATURES, load  # noqa: F401
from .attention import attention_with_cache_update, quantized_scaled_dot_product_attention  # noqa: F401
from .cache import (KVCacheSimple, MaskMode, QuantizedKVCache, RotatingKVCache, affine_dequantize,  # noqa: F401
                    affine_quantize, can_trim_prompt_cache, create_attention_mask,
                    KVCacheConfigurationError, make_attention_kv_cache, make_prompt_cache,
                    make_sliding_window_kv_cache,
                    maybe_affine_quantize_kv_cache, resolve_affine_scheme,
                    resolved_kv_quantization_group_size, trim_prompt_cache)
from .rounds import (AppendOnlyRoundStrategy, KVCacheRound, KVCacheRoundCommit, KVCacheStorage,  # noqa: F401
                     RotatingRestorePoint, RotatingRoundStrategy, RotatingStagedKVCache)
from .rope import RoPE, apply_rotary_position, attention_with_rope_and_cache_update  # noqa: F401
from .prefill import PrefillParameters  # noqa: F401
from .prompt_cache import KVCacheError, load_prompt_cache, save_prompt_cache  # noqa: F401
