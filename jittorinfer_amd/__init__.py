"""MI355X-native absorbed-MLA paged attention (GGML_OP_FLASH_ATTN_EXT, 576-d QK / 512-d V, and the latent-KV cache write that feeds it) behind the ggml
backend plugin interface.  The product is jittorinfer_amd/libggml-hip-mla.so (HIP kernels for gfx950, a thin C
ABI, and the ggml backend); this package is the Python host-side plumbing over that C ABI.  There is no CPU
fallback: every entry point raises if the library is missing."""
from .capi import (  # noqa: F401
    MLA_TYPE_BF16, MLA_TYPE_F16, MLA_TYPE_F32, MLA_TYPE_Q8_0, MLA_FLAG_F16_ACC_STRICT, MLA_FLAG_UNIFORM_SPLITS, MLA_FLAG_BF16_DIRECT, MLA_FLAG_MASK_EXTENTS_VALID, MLA_FLAG_Q8_EXACT,
    MlaAttnArgs, MlaPlanInfo, MlaKvWriteArgs, MlaRopeArgs, MlaMulMatArgs, MlaCopyArgs, library, library_path, ggml_flash_attn_ext,
    kv_write, plan, hbm_copy, PageTable, ggml_rope_ext, ggml_mul_mat, copy_f32, release_workspaces, FrontBatch,
)
