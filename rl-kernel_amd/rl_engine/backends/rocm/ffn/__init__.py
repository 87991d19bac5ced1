from rl_engine.backends.rocm.ffn.ffn import (  # noqa: F401
    BACKEND_ID,
    Qwen3FFNOp,
    qwen3_ffn,
    qwen3_ffn_packed_inference,
)
