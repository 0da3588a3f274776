"""The decoder the quantized Linear layers sit in (the unchanged caller of the
GEMM path): same modules, parameter names and math as the reference's
``astrai/model`` for a dense GQA + SwiGLU decoder, with a dense KV cache."""

from astrai_amd.model.decoder import (
    AutoRegressiveLM,
    AutoRegressiveLMConfig,
    DenseKVCache,
    fuse_int8_weights,
    greedy_generate,
    unfuse_int8_weights,
)

from astrai_amd.model.checkpoint import (load_fp8_scaling, load_int8_checkpoint, save_fp8_scaling,
                                         save_int8_checkpoint)

__all__ = ["load_fp8_scaling", "save_fp8_scaling", "load_int8_checkpoint", "save_int8_checkpoint", "AutoRegressiveLM", "AutoRegressiveLMConfig", "DenseKVCache", "greedy_generate",
           "fuse_int8_weights", "unfuse_int8_weights"]
