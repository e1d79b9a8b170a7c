"""Text in, text out: the tokenizer, the incremental text streamer and Gpt2Runtime over the
HIP backend.

Host-side only.  The token ids go through the same C-ABI entry points as everything else
(`pg_gpt2_stream_token_ids_with_stats` / `_profiled`); this module adds what the reference's
runtime wraps around them: `tokenizer.json` handling (src/models/gpt2/rust.rs:268-323),
IncrementalTextStreamer (src/models/streaming.rs:17-80) and the text entry points of
Gpt2Runtime (src/models/gpt2/rust.rs:325-634).  The tokenizer is the `tokenizers` package,
the Python binding of the crate the reference links; there is no substitute when it is
missing.
"""
from __future__ import annotations

import os
import time
import unicodedata
from typing import Callable, List, Optional, Sequence, Tuple

from .gpt2 import (GenerationStats, Gpt2Error, Gpt2GenerationConfig, Gpt2HipConfig, Gpt2Model,
                   Gpt2OperationProfile, TextGenerationConfig)

REPLACEMENT_CHARACTER = "�"


def escape_raw_token(token: str) -> str:
    """escape_raw_token (src/models/streaming.rs:17-30): one token per line of a raw-token
    stream; backslash, tab, newline, carriage return and other control characters escaped."""
    out = []
    for ch in token:
        if ch == "\\":
            out.append("\\\\")
        elif ch == "\t":
            out.append("\\t")
        elif ch == "\n":
            out.append("\\n")
        elif ch == "\r":
            out.append("\\r")
        elif unicodedata.category(ch) == "Cc":
            out.append("\\u{%x}" % ord(ch))
        else:
            out.append(ch)
    return "".join(out)


def is_incremental_decode_safe(token_text: str) -> bool:
    """is_incremental_decode_safe (src/models/streaming.rs:78-80): a token's own text may be
    emitted as it is unless it is empty or holds U+FFFD (a piece of a multi-byte character)."""
    return token_text != "" and REPLACEMENT_CHARACTER not in token_text


class IncrementalTextStreamer:
    """IncrementalTextStreamer (src/models/streaming.rs:32-76).  `decoder` is anything with
    `decode_tokens(ids) -> str` (the TokenDecoder trait, streaming.rs:1-9)."""

    def __init__(self, decoded: str = ""):
        self._decoded = decoded

    def decoded(self) -> str:
        return self._decoded

    def stream_token(self, decoder, output_ids: Sequence[int], token_id: int,
                     on_text: Callable[[str], None]) -> None:
        token_text = decoder.decode_tokens([token_id])
        if is_incremental_decode_safe(token_text):
            on_text(token_text)
            self._decoded += token_text
            return
        # Unsafe piece: decode everything and emit what is new against what was emitted.
        next_decoded = decoder.decode_tokens(output_ids)
        if next_decoded.startswith(self._decoded):
            on_text(next_decoded[len(self._decoded):])
        else:
            on_text(token_text)
        self._decoded = next_decoded


class Gpt2Tokenizer:
    """Gpt2Tokenizer (src/models/gpt2/rust.rs:268-323) over a `tokenizer.json`."""

    def __init__(self, tokenizer):
        self._tok = tokenizer

    @classmethod
    def from_file(cls, path) -> "Gpt2Tokenizer":
        try:
            from tokenizers import Tokenizer
        except ImportError as e:  # no stand-in: the text entry points need the real thing
            raise Gpt2Error("Asset", f"failed to load tokenizer {path}: the tokenizers package is missing ({e})")
        try:
            return cls(Tokenizer.from_file(os.fspath(path)))
        except Exception as e:
            raise Gpt2Error("Asset", f"failed to load tokenizer {path}: {e}")

    def encode(self, text: str) -> List[int]:
        try:
            return [int(i) for i in self._tok.encode(text, add_special_tokens=True).ids]
        except Exception as e:
            raise Gpt2Error("Asset", f"failed to encode prompt: {e}")

    def decode(self, token_ids: Sequence[int]) -> str:
        ids = [int(i) for i in token_ids]
        if any(i < 0 or i > 0xFFFFFFFF for i in ids):
            raise Gpt2Error("InvalidInput", "token id does not fit in u32")
        try:
            return self._tok.decode(ids, skip_special_tokens=True)
        except Exception as e:
            raise Gpt2Error("Asset", f"failed to decode tokens: {e}")

    # TokenDecoder / RawTokenDecoder (src/models/streaming.rs:1-15)
    decode_tokens = decode

    def decode_token(self, token_id: int) -> str:
        return self.decode([token_id])

    def raw_token(self, token_id: int) -> str:
        if token_id < 0 or token_id > 0xFFFFFFFF:
            raise Gpt2Error("InvalidInput", "token id does not fit in u32")
        tok = self._tok.id_to_token(int(token_id))
        if tok is None:
            raise Gpt2Error("InvalidInput", f"unknown token id {token_id}")
        return tok


class Gpt2Runtime:
    """Gpt2Runtime (src/models/gpt2/rust.rs:325-634): a model on the HIP backend plus its
    tokenizer.  Every generation below runs on the device through the C-ABI; the tokenizer and
    the streamer run on the host between token callbacks, as in the reference."""

    def __init__(self, model: Gpt2Model, tokenizer: Gpt2Tokenizer):
        self.model = model
        self.tokenizer = tokenizer

    @classmethod
    def from_dir(cls, model_dir, hip_config: Optional[Gpt2HipConfig] = None) -> "Gpt2Runtime":
        """from_dir_with_backend (rust.rs:382-393): config.json, model.safetensors,
        tokenizer.json of one directory (src/models/gpt2/assets.rs:20-28)."""
        model = Gpt2Model.from_dir(model_dir, hip_config)
        tokenizer = Gpt2Tokenizer.from_file(os.path.join(os.fspath(model_dir), "tokenizer.json"))
        return cls(model, tokenizer)

    def generate_greedy_text(self, prompt: str, max_new_tokens: int) -> str:
        """rust.rs:398-404."""
        input_ids = self.tokenizer.encode(prompt)
        return self.tokenizer.decode(self.model.generate_greedy_cached(input_ids, max_new_tokens))

    def stream_greedy_text(self, prompt: str, max_new_tokens: int,
                           on_text: Callable[[str], None]) -> str:
        """rust.rs:406-430: the prompt's text first, then every token's text as it is chosen."""
        input_ids = self.tokenizer.encode(prompt)
        output_ids = list(input_ids)
        streamer = IncrementalTextStreamer(self.tokenizer.decode(output_ids))
        on_text(streamer.decoded())

        def on_token(token_id: int) -> None:
            output_ids.append(token_id)
            streamer.stream_token(self.tokenizer, output_ids, token_id, on_text)

        self.model.stream_greedy_tokens(input_ids, max_new_tokens, on_token)
        return streamer.decoded()

    def stream_greedy_text_with_stats(self, prompt: str, max_new_tokens: int,
                                      on_text: Callable[[str], None]):
        """rust.rs:432-445."""
        return self.stream_text_with_stats(prompt, Gpt2GenerationConfig(max_new_tokens), on_text)

    def _check_generation(self, generation: TextGenerationConfig) -> None:
        generation.validate()
        eos = generation.eos_token_id
        if eos is not None and eos >= self.model.config.vocab_size:
            raise Gpt2Error("InvalidConfig",
                            f"generation eos_token_id {eos} is outside vocab_size {self.model.config.vocab_size}")

    def stream_text_with_stats(self, prompt: str, generation: TextGenerationConfig,
                               on_text: Callable[[str], None], profiled: bool = False
                               ) -> Tuple[str, GenerationStats, Gpt2OperationProfile]:
        """rust.rs:447-546.  Returns (text, stats, operation profile); the profile's
        `tokenization` and `decoding` buckets are host time, the other buckets are filled when
        `profiled` asks for the per-operation path."""
        self._check_generation(generation)
        t0 = time.perf_counter()
        input_ids = self.tokenizer.encode(prompt)
        tokenize_time = time.perf_counter() - t0

        output_ids = list(input_ids)
        t0 = time.perf_counter()
        decoded = self.tokenizer.decode(output_ids)
        decoding = time.perf_counter() - t0
        streamer = IncrementalTextStreamer(decoded)
        on_text(streamer.decoded())

        def on_token(token_id: int) -> None:
            nonlocal decoding
            output_ids.append(token_id)
            t = time.perf_counter()
            try:
                streamer.stream_token(self.tokenizer, output_ids, token_id, on_text)
            finally:
                decoding += time.perf_counter() - t

        _, stats, profile = self._run(input_ids, generation, on_token, profiled)
        stats.tokenize_time = tokenize_time
        profile.tokenization += tokenize_time
        profile.decoding += decoding
        return streamer.decoded(), stats, profile

    def stream_token_ids_with_stats(self, prompt: str, generation: TextGenerationConfig,
                                    on_token: Optional[Callable[[int], None]] = None,
                                    profiled: bool = False
                                    ) -> Tuple[List[int], GenerationStats, Gpt2OperationProfile]:
        """rust.rs:548-634: prompt ids followed by the generated ids."""
        self._check_generation(generation)
        t0 = time.perf_counter()
        input_ids = self.tokenizer.encode(prompt)
        tokenize_time = time.perf_counter() - t0
        tokens, stats, profile = self._run(input_ids, generation, on_token, profiled)
        stats.tokenize_time = tokenize_time
        profile.tokenization += tokenize_time
        return tokens, stats, profile

    def _run(self, input_ids, generation, on_token, profiled):
        if profiled:
            return self.model.stream_token_ids_with_stats(input_ids, generation, on_token, profiled=True)
        tokens, stats = self.model.stream_token_ids_with_stats(input_ids, generation, on_token)
        return tokens, stats, Gpt2OperationProfile()
