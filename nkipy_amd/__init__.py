"""MI355X-native paged flash attention behind nkipy's NumPy-style kernel convention."""
from .paged_attn import (PreparedStep, QTransform, blocksparse_prefill, check_block_tables, decode, decode_step, decode_workspace_bytes,
                         default_scale, gather_kv, kv_write, o_proj, o_proj_workspace_bytes, prefill, prepare_decode_step, prepare_verify_step,
                         qk_norm_rope_kv_write, rope_tables, verify, verify_step)

__all__ = ["decode", "decode_step", "prefill", "verify", "blocksparse_prefill", "gather_kv", "decode_workspace_bytes",
           "check_block_tables", "default_scale", "kv_write", "qk_norm_rope_kv_write", "rope_tables", "QTransform", "o_proj",
           "o_proj_workspace_bytes", "verify_step", "prepare_decode_step", "prepare_verify_step", "PreparedStep"]
