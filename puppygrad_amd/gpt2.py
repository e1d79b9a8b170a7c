"""Python host-side mirror of puppygrad's GPT-2 model/runtime API over the HIP C ABI.

Names, argument meaning and error behaviour follow the reference
(src/models/gpt2/rust.rs, src/models/autoregressive.rs, src/models/generation.rs)
so tests read like the reference's own: `Gpt2Model.new(config, weights)`,
`model.new_kv_cache()`, `model.prefill(ids, cache)`, `model.forward_one(id, cache)`,
`model.select_next_token(logits)`, `generate(model, ids, max_new, on_token)`.
All compute happens inside libpuppygrad_hip.so.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

import numpy as np

from . import _lib

GPT2_EOS_TOKEN_ID = 50_256  # src/models/gpt2/options.rs:8


class Gpt2Error(Exception):
    """Gpt2Error (src/models/gpt2/error.rs:4-21); `kind` is the variant name."""

    PREFIX = {
        "Asset": "GPT-2 asset error: ",
        "InvalidConfig": "invalid GPT-2 config: ",
        "InvalidInput": "invalid GPT-2 input: ",
        "InvalidWeights": "invalid GPT-2 weights: ",
        "Backend": "GPT-2 hip backend error: ",
    }

    def __init__(self, kind: str, msg: str):
        super().__init__(self.PREFIX[kind] + msg)
        self.kind = kind
        self.msg = msg


_KIND = {_lib.PG_ASSET: "Asset", _lib.PG_INVALID_CONFIG: "InvalidConfig",
         _lib.PG_INVALID_INPUT: "InvalidInput", _lib.PG_INVALID_WEIGHTS: "InvalidWeights",
         _lib.PG_BACKEND: "Backend"}


def _check(status: int) -> None:
    if status != _lib.PG_OK:
        msg = _lib.load().pg_last_error_message().decode()
        raise Gpt2Error(_KIND.get(status, "Backend"), msg)


@dataclass
class Gpt2Config:
    """Gpt2Config (src/models/gpt2/rust.rs:30-58)."""
    vocab_size: int
    n_positions: int
    n_embd: int
    n_layer: int
    n_head: int
    n_inner: Optional[int] = None
    layer_norm_epsilon: float = 1e-5

    def __post_init__(self):
        if self.n_inner is None:
            self.n_inner = 4 * self.n_embd

    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    def to_c(self) -> _lib.pg_gpt2_config:
        return _lib.pg_gpt2_config(self.vocab_size, self.n_positions, self.n_embd, self.n_layer,
                                   self.n_head, self.n_inner, self.layer_norm_epsilon)

    @classmethod
    def from_c(cls, c: _lib.pg_gpt2_config) -> "Gpt2Config":
        return cls(c.vocab_size, c.n_positions, c.n_embd, c.n_layer, c.n_head, c.n_inner,
                   c.layer_norm_epsilon)

    @classmethod
    def from_json_file(cls, path) -> "Gpt2Config":
        """load_config (src/models/gpt2/rust.rs:696-711): a Hugging Face config.json."""
        c = _lib.pg_gpt2_config()
        _check(_lib.load().pg_gpt2_load_config(str(path).encode(), C.byref(c)))
        return cls.from_c(c)


@dataclass
class Gpt2BlockWeights:
    """Gpt2BlockWeights (src/models/gpt2/rust.rs:111-125); matrices in HF [in,out] layout."""
    ln_1_g: np.ndarray
    ln_1_b: np.ndarray
    c_attn_w: np.ndarray
    c_attn_b: np.ndarray
    c_proj_w: np.ndarray
    c_proj_b: np.ndarray
    ln_2_g: np.ndarray
    ln_2_b: np.ndarray
    c_fc_w: np.ndarray
    c_fc_b: np.ndarray
    c_proj_mlp_w: np.ndarray
    c_proj_mlp_b: np.ndarray


@dataclass
class Gpt2Weights:
    """Gpt2Weights (src/models/gpt2/rust.rs:102-109): flat f32 arrays."""
    wte: np.ndarray
    wpe: np.ndarray
    blocks: List[Gpt2BlockWeights]
    ln_f_g: np.ndarray
    ln_f_b: np.ndarray


def _tensor(arr: np.ndarray, keep: list) -> _lib.pg_tensor:
    a = np.ascontiguousarray(arr, dtype=np.float32).reshape(-1)
    keep.append(a)
    return _lib.pg_tensor(_lib.f32p(a), a.size)


def weights_view(weights: Gpt2Weights, keep: list) -> _lib.pg_gpt2_weights_view:
    """Build the C view; `keep` receives the arrays that must outlive the call."""
    blocks = (_lib.pg_gpt2_block_view * max(len(weights.blocks), 1))()
    for i, b in enumerate(weights.blocks):
        for name in _lib.BLOCK_FIELDS:
            setattr(blocks[i], name, _tensor(getattr(b, name), keep))
    keep.append(blocks)
    return _lib.pg_gpt2_weights_view(_tensor(weights.wte, keep), _tensor(weights.wpe, keep),
                                     _tensor(weights.ln_f_g, keep), _tensor(weights.ln_f_b, keep),
                                     C.cast(blocks, C.POINTER(_lib.pg_gpt2_block_view)),
                                     len(weights.blocks))


class TensorStore:
    """TensorStore (src/models/safetensors.rs:93-138) over a mapped .safetensors file.
    Arrays returned are read-only views into the mapping and keep the store alive."""

    def __init__(self, path):
        h = C.c_void_p()
        _check(_lib.load().pg_tensor_store_open(str(path).encode(), C.byref(h)))
        self._h = h

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            _lib.load().pg_tensor_store_close(h)
            self._h = None

    def __len__(self) -> int:
        return int(_lib.load().pg_tensor_store_len(self._h))

    def _view(self, t: _lib.pg_tensor, shape) -> np.ndarray:
        n = int(t.len)
        if n == 0:
            arr = np.zeros(0, np.float32)
        else:
            addr = C.cast(t.data, C.c_void_p).value
            arr = np.frombuffer((C.c_float * n).from_address(addr), np.float32)
        arr = arr.reshape(tuple(shape))
        arr.flags.writeable = False  # the mapping is read-only
        return _StoreArray.wrap(arr, self)

    def required_f32(self, name: str, expected_shape: Sequence[int]) -> np.ndarray:
        shape = (C.c_uint64 * max(len(expected_shape), 1))(*expected_shape)
        t = _lib.pg_tensor()
        _check(_lib.load().pg_tensor_store_required_f32(self._h, name.encode(), shape,
                                                        len(expected_shape), C.byref(t)))
        return self._view(t, expected_shape)

    def optional_f32(self, name: str, expected_shape: Sequence[int]) -> Optional[np.ndarray]:
        shape = (C.c_uint64 * max(len(expected_shape), 1))(*expected_shape)
        t = _lib.pg_tensor()
        found = C.c_int32(0)
        _check(_lib.load().pg_tensor_store_optional_f32(self._h, name.encode(), shape,
                                                        len(expected_shape), C.byref(found),
                                                        C.byref(t)))
        return self._view(t, expected_shape) if found.value else None


class _StoreArray(np.ndarray):
    """An ndarray that holds a reference to the TensorStore whose mapping it views."""

    @classmethod
    def wrap(cls, arr: np.ndarray, store: TensorStore) -> "np.ndarray":
        out = arr.view(cls)
        out._store = store
        return out

    def __array_finalize__(self, obj):
        self._store = getattr(obj, "_store", None)


def load_weights(path, cfg: Gpt2Config) -> Gpt2Weights:
    """load_weights (src/models/gpt2/rust.rs:713-771) into host arrays: Hugging Face tensor
    names, each tried bare and then with the `transformer.` prefix.  (Gpt2Model.from_dir
    does the same inside the library without host copies.)"""
    store = TensorStore(path)

    def tensor(name: str, shape) -> np.ndarray:
        found = store.optional_f32(name, shape)
        return found if found is not None else store.required_f32("transformer." + name, shape)

    c, i = cfg.n_embd, cfg.n_inner
    blocks = []
    for layer in range(cfg.n_layer):
        p = f"h.{layer}"
        blocks.append(Gpt2BlockWeights(
            ln_1_g=tensor(f"{p}.ln_1.weight", [c]), ln_1_b=tensor(f"{p}.ln_1.bias", [c]),
            c_attn_w=tensor(f"{p}.attn.c_attn.weight", [c, 3 * c]),
            c_attn_b=tensor(f"{p}.attn.c_attn.bias", [3 * c]),
            c_proj_w=tensor(f"{p}.attn.c_proj.weight", [c, c]),
            c_proj_b=tensor(f"{p}.attn.c_proj.bias", [c]),
            ln_2_g=tensor(f"{p}.ln_2.weight", [c]), ln_2_b=tensor(f"{p}.ln_2.bias", [c]),
            c_fc_w=tensor(f"{p}.mlp.c_fc.weight", [c, i]), c_fc_b=tensor(f"{p}.mlp.c_fc.bias", [i]),
            c_proj_mlp_w=tensor(f"{p}.mlp.c_proj.weight", [i, c]),
            c_proj_mlp_b=tensor(f"{p}.mlp.c_proj.bias", [c])))
    return Gpt2Weights(wte=tensor("wte.weight", [cfg.vocab_size, c]),
                       wpe=tensor("wpe.weight", [cfg.n_positions, c]), blocks=blocks,
                       ln_f_g=tensor("ln_f.weight", [c]), ln_f_b=tensor("ln_f.bias", [c]))


@dataclass
class Gpt2HipConfig:
    """The per-backend knobs that sit where Gpt2RustConfig does
    (src/models/gpt2/options.rs:54-96)."""
    device: int = 0
    weight_storage: int = _lib.PG_STORE_F32
    decode_path: int = _lib.PG_DECODE_AUTO
    prefill_path: int = 0  # 0: GEMM prefill for prompts of seq_gemm_min_tokens and more, 1: token by token
    # tunables (0 = built-in default): what the autotune scan varies and puppygrad-tune.json holds
    attn_item_keys: int = 0
    attn_blocks_per_cu: int = 0
    gemm_split_items_per_cu: int = 0
    gemm_b9_min_rows: int = 0
    seq_gemm_min_tokens: int = 0

    def to_c(self) -> _lib.pg_hip_options:
        return _lib.pg_hip_options(self.device, self.weight_storage, self.decode_path,
                                   self.prefill_path, self.attn_item_keys, self.attn_blocks_per_cu,
                                   self.gemm_split_items_per_cu, self.gemm_b9_min_rows,
                                   self.seq_gemm_min_tokens, 0)


@dataclass
class TextGenerationConfig:
    """TextGenerationConfig (src/models/generation.rs:61-89)."""
    max_new_tokens: int
    eos_token_id: Optional[int] = None
    temperature: float = 0.0
    top_p: Optional[float] = None
    top_k: Optional[int] = None
    seed: int = 299_792_458
    repeat_penalty: float = 1.0
    repeat_last_n: int = 128

    def to_c(self) -> _lib.pg_sampling:
        return _lib.pg_sampling(self.temperature, int(self.top_p is not None),
                                self.top_p if self.top_p is not None else 0.0,
                                int(self.top_k is not None),
                                self.top_k if self.top_k is not None else 0,
                                self.repeat_penalty, self.repeat_last_n)

    def validate(self) -> None:
        s = self.to_c()
        _check(_lib.load().pg_sampling_validate(C.byref(s)))


def Gpt2GenerationConfig(max_new_tokens: int) -> TextGenerationConfig:
    """Gpt2GenerationConfig::new (src/models/gpt2/options.rs:156-162): EOS 50256."""
    return TextGenerationConfig(max_new_tokens, eos_token_id=GPT2_EOS_TOKEN_ID)


@dataclass
class Gpt2OperationProfile:
    """Gpt2OperationProfile (src/models/gpt2/rust.rs:336-347), seconds per bucket.  LayerNorm
    runs inside the projection that consumes it on this backend: its bucket stays 0."""
    tokenization: float = 0.0
    layer_norm: float = 0.0
    qkv_projection: float = 0.0
    attention: float = 0.0
    attention_projection: float = 0.0
    mlp_fc_projection: float = 0.0
    mlp_projection: float = 0.0
    final_logits: float = 0.0
    decoding: float = 0.0


@dataclass
class GenerationStats:
    """GenerationStats (src/models/generation.rs:129-180)."""
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefill_time: float = 0.0
    decode_time: float = 0.0
    first_token_time: Optional[float] = None
    gpu_decode_time: float = 0.0
    tokenize_time: float = 0.0  # host time of the prompt's encode; set by Gpt2Runtime

    @property
    def total_generation_time(self) -> float:
        return self.prefill_time + self.decode_time

    def total_model_tokens(self) -> int:
        return self.prompt_tokens + self.generated_tokens

    @staticmethod
    def _rate(tokens: int, seconds: float) -> float:
        return 0.0 if seconds == 0.0 else tokens / seconds

    def prefill_tokens_per_second(self) -> float:
        return self._rate(self.prompt_tokens, self.prefill_time)

    def decode_tokens_per_second(self) -> float:
        return self._rate(self.generated_tokens, self.decode_time)

    def total_tokens_per_second(self) -> float:
        return self._rate(self.total_model_tokens(), self.total_generation_time)

    def average_decode_token_time(self) -> Optional[float]:
        if self.generated_tokens == 0:
            return None
        return self.decode_time / self.generated_tokens


def _u32(ids: Sequence[int]) -> np.ndarray:
    arr = np.asarray(ids, dtype=np.int64).reshape(-1)
    if arr.size and (arr.min() < 0 or arr.max() > 0xFFFFFFFF):
        raise Gpt2Error("InvalidInput", "token id out of u32 range")
    return arr.astype(np.uint32)


class DeviceLogits:
    """The `Logits` associated type of the HIP decoder: a device-resident buffer
    owned by its cache, valid until the next call that takes that cache."""

    def __init__(self, handle: int, cache: "Gpt2KvCache"):
        self._h = handle
        self._cache = cache

    @property
    def rows(self) -> int:
        return _lib.load().pg_logits_rows(self._h)

    @property
    def vocab(self) -> int:
        return _lib.load().pg_logits_vocab(self._h)

    def to_host(self) -> np.ndarray:
        out = np.empty((self.rows, self.vocab), dtype=np.float32)
        _check(_lib.load().pg_logits_copy_to_host(self._h, _lib.f32p(out), out.size))
        return out[0] if self.rows == 1 else out

    def argmax(self) -> np.ndarray:
        out = np.empty(self.rows, dtype=np.uint32)
        _check(_lib.load().pg_logits_argmax(self._h, _lib.u32p(out)))
        return out


class Gpt2KvCache:
    """Gpt2KvCache (src/models/gpt2/rust.rs:177-249) living in HBM."""

    def __init__(self, model: "Gpt2Model", batch: int = 1):
        h = C.c_void_p()
        _check(_lib.load().pg_kv_cache_create(model._h, batch, C.byref(h)))
        self._h = h
        self._model = model  # keeps the model alive

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            _lib.load().pg_kv_cache_destroy(h)
            self._h = None

    @property
    def seq_len(self) -> int:
        return _lib.load().pg_kv_cache_seq_len(self._h)

    @seq_len.setter
    def seq_len(self, n: int) -> None:
        _check(_lib.load().pg_kv_cache_set_seq_len(self._h, n))

    @property
    def max_seq_len(self) -> int:
        return _lib.load().pg_kv_cache_max_seq_len(self._h)

    @property
    def batch(self) -> int:
        return _lib.load().pg_kv_cache_batch(self._h)

    def clear(self) -> None:
        _check(_lib.load().pg_kv_cache_clear(self._h))

    def read_layer(self, layer: int, which: int, b: int = 0) -> np.ndarray:
        cfg = self._model.config
        out = np.empty((cfg.n_head, cfg.n_positions, cfg.head_dim()), dtype=np.float32)
        _check(_lib.load().pg_kv_cache_read_layer(self._h, b, layer, which, _lib.f32p(out),
                                                  out.size))
        return out


class Gpt2Model:
    """Gpt2Model (src/models/gpt2/rust.rs:141-148, 798-1051) on the HIP backend;
    implements AutoregressiveDecoder (src/models/autoregressive.rs:9-31)."""

    def __init__(self, handle, config: Gpt2Config):
        self._h = handle
        self.config = config

    @classmethod
    def new(cls, config: Gpt2Config, weights: Gpt2Weights,
            hip_config: Optional[Gpt2HipConfig] = None) -> "Gpt2Model":
        keep: list = []
        cfg = config.to_c()
        view = weights_view(weights, keep)
        opts = (hip_config or Gpt2HipConfig()).to_c()
        h = C.c_void_p()
        _check(_lib.load().pg_gpt2_create(C.byref(cfg), C.byref(view), C.byref(opts), C.byref(h)))
        return cls(h, config)

    @classmethod
    def from_dir(cls, model_dir, hip_config: Optional[Gpt2HipConfig] = None) -> "Gpt2Model":
        """Gpt2Runtime::from_dir_with_backend without the tokenizer
        (src/models/gpt2/rust.rs:382-393): `config.json` + `model.safetensors`."""
        opts = (hip_config or Gpt2HipConfig()).to_c()
        h = C.c_void_p()
        lib = _lib.load()
        _check(lib.pg_gpt2_create_from_dir(str(model_dir).encode(), C.byref(opts), C.byref(h)))
        cfg = _lib.pg_gpt2_config()
        _check(lib.pg_gpt2_get_config(h, C.byref(cfg)))
        return cls(h, Gpt2Config.from_c(cfg))

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            _lib.load().pg_gpt2_destroy(h)
            self._h = None

    def describe(self) -> str:
        buf = C.create_string_buffer(256)
        _check(_lib.load().pg_gpt2_describe(self._h, buf, len(buf)))
        return buf.value.decode()

    # -- AutoregressiveDecoder -------------------------------------------------
    def max_context_len(self) -> int:
        return self.config.n_positions

    def new_kv_cache(self, batch: int = 1) -> Gpt2KvCache:
        return Gpt2KvCache(self, batch)

    new_cache = new_kv_cache

    def prefill(self, input_ids: Sequence[int], cache: Gpt2KvCache) -> DeviceLogits:
        ids = _u32(input_ids)
        out = C.c_void_p()
        _check(_lib.load().pg_gpt2_prefill(self._h, cache._h, _lib.u32p(ids), ids.size,
                                           C.byref(out)))
        return DeviceLogits(out, cache)

    def prefill_profiled(self, input_ids: Sequence[int], cache: Gpt2KvCache):
        """prefill_profiled (rust.rs:906-927): the logits and the per-operation times."""
        ids = _u32(input_ids)
        out = C.c_void_p()
        prof = _lib.pg_gpt2_operation_profile()
        _check(_lib.load().pg_gpt2_prefill_profiled(self._h, cache._h, _lib.u32p(ids), ids.size,
                                                    C.byref(out), C.byref(prof)))
        return DeviceLogits(out, cache), Gpt2OperationProfile(
            **{f[0][:-2]: getattr(prof, f[0]) for f in prof._fields_})

    def forward_one(self, token_id: int, cache: Gpt2KvCache) -> DeviceLogits:
        if token_id < 0 or token_id > 0xFFFFFFFF:
            raise Gpt2Error("InvalidInput", f"token id {token_id} exceeds vocab_size "
                                            f"{self.config.vocab_size}")
        out = C.c_void_p()
        _check(_lib.load().pg_gpt2_forward_one(self._h, cache._h, token_id, C.byref(out)))
        return DeviceLogits(out, cache)

    def select_next_token(self, logits: DeviceLogits) -> int:
        return int(logits.argmax()[0])

    # -- batched forms ---------------------------------------------------------
    def prefill_batch(self, input_ids: np.ndarray, cache: Gpt2KvCache) -> DeviceLogits:
        ids = np.ascontiguousarray(np.asarray(input_ids, dtype=np.uint32))
        if ids.ndim != 2 or ids.shape[0] != cache.batch:
            raise Gpt2Error("InvalidInput", "prefill_batch expects ids of shape [batch][n]")
        out = C.c_void_p()
        _check(_lib.load().pg_gpt2_prefill_batch(self._h, cache._h, _lib.u32p(ids), ids.shape[1],
                                                 C.byref(out)))
        return DeviceLogits(out, cache)

    def forward_one_batch(self, token_ids: Sequence[int], cache: Gpt2KvCache) -> DeviceLogits:
        ids = _u32(token_ids)
        if ids.size != cache.batch:
            raise Gpt2Error("InvalidInput", "forward_one_batch expects one id per sequence")
        out = C.c_void_p()
        _check(_lib.load().pg_gpt2_forward_one_batch(self._h, cache._h, _lib.u32p(ids),
                                                     C.byref(out)))
        return DeviceLogits(out, cache)

    # -- full-sequence forward (rust.rs:831-882) ---------------------------------
    def forward(self, input_ids: Sequence[int]) -> "Gpt2Output":
        ids = _u32(input_ids)
        out = np.empty((max(ids.size, 1), self.config.vocab_size), dtype=np.float32)
        _check(_lib.load().pg_gpt2_forward(self._h, _lib.u32p(ids), ids.size, _lib.f32p(out),
                                           ids.size * self.config.vocab_size))
        return Gpt2Output(out[:ids.size], ids.size, self.config.vocab_size)

    # -- generation (rust.rs:884-900, 1008-1027) ---------------------------------
    def generate_greedy(self, input_ids: Sequence[int], max_new_tokens: int) -> List[int]:
        """generate_greedy: a full forward per new token (rust.rs:884-900)."""
        tokens = [int(t) for t in input_ids]
        _check_nonempty(tokens)
        for _ in range(max_new_tokens):
            if len(tokens) >= self.config.n_positions:
                break
            out = self.forward(tokens)
            tokens.append(argmax_logits(out.last_logits()))
        return tokens

    def generate_greedy_cached(self, input_ids: Sequence[int], max_new_tokens: int) -> List[int]:
        return self.stream_greedy_tokens(input_ids, max_new_tokens, lambda _t: None)

    def stream_greedy_tokens(self, input_ids: Sequence[int], max_new_tokens: int,
                             on_token: Callable[[int], None]) -> List[int]:
        return generate(self, input_ids, max_new_tokens, on_token)

    def decode_greedy(self, cache: Gpt2KvCache, max_new: int,
                      eos: Optional[int] = None) -> "tuple[List[int], GenerationStats]":
        """The greedy loop with the token kept on the device (pg_gpt2_decode_greedy)."""
        out = np.empty(max(max_new, 1), dtype=np.uint32)
        n = C.c_uint32()
        st = _lib.pg_generation_stats()
        _check(_lib.load().pg_gpt2_decode_greedy(self._h, cache._h, max_new,
                                                 -1 if eos is None else eos, _lib.u32p(out),
                                                 C.byref(n), C.byref(st)))
        return [int(t) for t in out[:n.value]], _stats(st)

    def decode_greedy_batch(self, cache: Gpt2KvCache,
                            steps: int) -> "tuple[np.ndarray, GenerationStats]":
        out = np.empty((max(steps, 1), cache.batch), dtype=np.uint32)
        st = _lib.pg_generation_stats()
        _check(_lib.load().pg_gpt2_decode_greedy_batch(self._h, cache._h, steps, _lib.u32p(out),
                                                       C.byref(st)))
        return out[:st.generated_tokens], _stats(st)

    def stream_token_ids_with_stats(self, input_ids: Sequence[int],
                                    generation: TextGenerationConfig,
                                    on_token: Optional[Callable[[int], None]] = None,
                                    profiled: bool = False):
        """Gpt2Runtime::stream_token_ids_with_stats with ids in place of a prompt
        string (rust.rs:548-634).  With profiled=True every forward runs as one launch per
        operation, timed into a Gpt2OperationProfile, and a third value is returned."""
        ids = _u32(input_ids)
        out = np.empty(ids.size + generation.max_new_tokens + 1, dtype=np.uint32)
        n = C.c_size_t()
        st = _lib.pg_generation_stats()
        samp = generation.to_c()
        err: list = []

        def _cb(tok, _user):
            try:
                if on_token is not None:
                    on_token(int(tok))
                return 0
            except Exception as e:  # surfaced after the C call returns
                err.append(e)
                return 1

        cb = _lib.ON_TOKEN(_cb)
        args = (self._h, _lib.u32p(ids), ids.size, generation.max_new_tokens,
                -1 if generation.eos_token_id is None else generation.eos_token_id, C.byref(samp),
                generation.seed, cb, None, _lib.u32p(out), C.byref(n), C.byref(st))
        prof = _lib.pg_gpt2_operation_profile()
        if profiled:
            status = _lib.load().pg_gpt2_stream_token_ids_profiled(*args, C.byref(prof))
        else:
            status = _lib.load().pg_gpt2_stream_token_ids_with_stats(*args)
        if err:
            raise err[0]
        _check(status)
        tokens = [int(t) for t in out[:n.value]]
        if profiled:
            return tokens, _stats(st), Gpt2OperationProfile(
                **{f[0][:-2]: getattr(prof, f[0]) for f in prof._fields_})
        return tokens, _stats(st)


def _stats(st: _lib.pg_generation_stats) -> GenerationStats:
    return GenerationStats(st.prompt_tokens, st.generated_tokens, st.prefill_s, st.decode_s,
                           st.first_token_s if st.first_token_s >= 0 and st.generated_tokens else None,
                           st.gpu_decode_s)


def _check_nonempty(tokens) -> None:
    if len(tokens) == 0:
        raise Gpt2Error("InvalidInput", "input_ids must not be empty")


@dataclass
class Gpt2Output:
    """Gpt2Output (src/models/gpt2/rust.rs:150-175)."""
    logits: np.ndarray
    seq_len: int
    vocab_size: int

    def logits_for_position(self, pos: int) -> np.ndarray:
        if pos >= self.seq_len:
            raise Gpt2Error("InvalidInput",
                            f"position {pos} out of range for seq_len {self.seq_len}")
        return self.logits[pos]

    def last_logits(self) -> np.ndarray:
        if self.seq_len == 0:
            raise Gpt2Error("InvalidInput", "empty sequence")
        return self.logits_for_position(self.seq_len - 1)


def argmax_logits(values: np.ndarray) -> int:
    """argmax_logits (src/models/generation.rs:269-279) on a host vector, computed
    on the device through pg_op_argmax."""
    v = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
    out = C.c_uint32()
    _check(_lib.load().pg_op_argmax(0, _lib.f32p(v), v.size, C.byref(out)))
    return int(out.value)


def generate(model, input_ids: Sequence[int], max_new_tokens: int,
             on_token: Callable[[int], None]) -> List[int]:
    """autoregressive::generate (src/models/autoregressive.rs:61-87)."""
    cache = model.new_cache()
    logits = model.prefill(input_ids, cache)
    tokens = [int(t) for t in input_ids]
    for _ in range(max_new_tokens):
        if len(tokens) >= model.max_context_len():
            break
        nxt = model.select_next_token(logits)
        tokens.append(nxt)
        on_token(nxt)
        logits = model.forward_one(nxt, cache)
    return tokens


class LogitsSampler:
    """LogitsSampler (src/models/generation.rs:209-241) over device logits."""

    def __init__(self, seed: int):
        self._rng = _lib.pg_rng_state()
        _lib.load().pg_rng_seed(C.byref(self._rng), seed)

    def select_next_token(self, logits: DeviceLogits, history: Sequence[int],
                          config: TextGenerationConfig, row: int = 0) -> int:
        hist = _u32(history)
        samp = config.to_c()
        out = C.c_uint32()
        _check(_lib.load().pg_logits_sample(logits._h, row, _lib.u32p(hist), hist.size,
                                            C.byref(samp), C.byref(self._rng), C.byref(out)))
        return int(out.value)
