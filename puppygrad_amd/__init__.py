"""puppygrad_amd: MI355X (gfx950) GPT-2 inference backend for puppygrad.

The product is libpuppygrad_hip.so (C ABI in include/puppygrad_hip.h); this
package is its Python host-side mirror, used by the tests and the benchmark.
"""
from .gpt2 import (GPT2_EOS_TOKEN_ID, DeviceLogits, GenerationStats, Gpt2BlockWeights, Gpt2Config,
                   Gpt2Error, Gpt2GenerationConfig, Gpt2HipConfig, Gpt2KvCache, Gpt2Model,
                   Gpt2OperationProfile, Gpt2Output, Gpt2Weights, LogitsSampler, TensorStore, TextGenerationConfig,
                   argmax_logits, generate, load_weights)
from .runtime import (Gpt2Runtime, Gpt2Tokenizer, IncrementalTextStreamer, escape_raw_token,
                      is_incremental_decode_safe)

__all__ = ["GPT2_EOS_TOKEN_ID", "DeviceLogits", "GenerationStats", "Gpt2BlockWeights",
           "Gpt2Config", "Gpt2Error", "Gpt2GenerationConfig", "Gpt2HipConfig", "Gpt2KvCache",
           "Gpt2Model", "Gpt2OperationProfile", "Gpt2Output", "Gpt2Runtime", "Gpt2Tokenizer", "Gpt2Weights",
           "IncrementalTextStreamer", "LogitsSampler", "TensorStore", "escape_raw_token",
           "is_incremental_decode_safe",
           "TextGenerationConfig", "argmax_logits", "generate", "load_weights"]
