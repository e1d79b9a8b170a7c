"""The text side of Gpt2Runtime: incremental text streaming (src/models/streaming.rs), the
tokenizer wrapper and the text entry points (src/models/gpt2/rust.rs:268-634).

The streamer's known answers are the reference's own (streaming.rs:82-148).  There is no
`tokenizer.json` of a real checkpoint here: the tests train a small byte-level BPE with the
`tokenizers` package (the format and the decoder GPT-2's own file uses) and write it next to a
seeded model."""
import pytest

import oracle
from puppygrad_amd import (Gpt2Config, Gpt2Error, Gpt2Runtime, Gpt2Tokenizer, IncrementalTextStreamer,
                           TextGenerationConfig, escape_raw_token, is_incremental_decode_safe, synth)
from test_assets import write_model_dir

CORPUS = ["the quick brown fox jumps over the lazy dog", "hello world, hello there",
          "a stream of tokens becomes a stream of text", "naïve café — déjà vu", "🙂 smile 🙂"]
VOCAB = 300


class MockDecoder:
    """The decoder of streaming.rs:85-101."""

    def decode_tokens(self, token_ids):
        return "".join({0: "hello", 1: " world", 2: ""}.get(t, "�") for t in token_ids)


def collect(streamer, decoder, output_ids, token_id):
    chunks = []
    streamer.stream_token(decoder, output_ids, token_id, chunks.append)
    return chunks


def test_streams_safe_token_text_incrementally():
    s = IncrementalTextStreamer("hello")
    assert collect(s, MockDecoder(), [0, 1], 1) == [" world"]
    assert s.decoded() == "hello world"


def test_falls_back_to_full_decode_for_unsafe_token_text():
    s = IncrementalTextStreamer("hello")
    assert collect(s, MockDecoder(), [0, 1, 2], 2) == [" world"]
    assert s.decoded() == "hello world"


def test_emits_the_token_text_when_the_full_decode_does_not_extend_what_was_emitted():
    s = IncrementalTextStreamer("other")
    assert collect(s, MockDecoder(), [0, 3], 3) == ["�"]
    assert s.decoded() == "hello�"


def test_incremental_decode_rejects_empty_and_replacement_text():
    assert is_incremental_decode_safe(" hello")
    assert not is_incremental_decode_safe("")
    assert not is_incremental_decode_safe("�")
    assert not is_incremental_decode_safe("a�")


def test_escapes_raw_tokens_for_line_streams():
    assert escape_raw_token("<|en|>") == "<|en|>"
    assert escape_raw_token("ĠI") == "ĠI"
    assert escape_raw_token("a\tb\nc") == "a\\tb\\nc"
    assert escape_raw_token("a\\b\r") == "a\\\\b\\r"
    assert escape_raw_token("\x07\x7f") == "\\u{7}\\u{7f}"


def write_tokenizer(path):
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers, trainers
    tok = Tokenizer(models.BPE())
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tok.decoder = decoders.ByteLevel()
    trainer = trainers.BpeTrainer(vocab_size=VOCAB, special_tokens=[], show_progress=False,
                                  initial_alphabet=pre_tokenizers.ByteLevel.alphabet())
    tok.train_from_iterator(CORPUS, trainer)
    assert tok.get_vocab_size() <= VOCAB
    tok.save(str(path))
    return path


@pytest.fixture(scope="module")
def tokenizer(tmp_path_factory):
    return Gpt2Tokenizer.from_file(write_tokenizer(tmp_path_factory.mktemp("tok") / "tokenizer.json"))


def test_tokenizer_round_trips_text_and_names_raw_tokens(tokenizer):
    for text in CORPUS + ["tabs\tand\nlines", ""]:
        ids = tokenizer.encode(text)
        assert all(0 <= i < VOCAB for i in ids)
        assert tokenizer.decode(ids) == text
    ids = tokenizer.encode(" dog")
    assert tokenizer.raw_token(ids[0]).startswith("Ġ")  # byte-level spelling of the space
    assert tokenizer.decode_token(ids[0]).startswith(" ")
    with pytest.raises(Gpt2Error, match="unknown token id 100000"):
        tokenizer.raw_token(100000)
    with pytest.raises(Gpt2Error, match="token id does not fit in u32"):
        tokenizer.decode([1 << 32])


def test_tokenizer_load_failure_is_an_asset_error(tmp_path):
    with pytest.raises(Gpt2Error, match="failed to load tokenizer") as e:
        Gpt2Tokenizer.from_file(tmp_path / "tokenizer.json")
    assert e.value.kind == "Asset"
    (tmp_path / "tokenizer.json").write_text("{not json")
    with pytest.raises(Gpt2Error, match="failed to load tokenizer"):
        Gpt2Tokenizer.from_file(tmp_path / "tokenizer.json")


@pytest.mark.parametrize("text", ["hello world, the lazy dog", "café 🙂 déjà", "🙂🙂"])
def test_streamer_over_byte_level_tokens_ends_on_the_full_decode(tokenizer, text):
    """Multi-byte characters split over tokens decode to U+FFFD piece by piece: those pieces take
    the full-decode route, and whatever was emitted on the way the streamer's text ends equal to
    the decode of all ids.  Plain ASCII streams as the exact pieces."""
    ids = tokenizer.encode(text)
    s = IncrementalTextStreamer("")
    chunks, out = [], []
    for t in ids:
        out.append(t)
        s.stream_token(tokenizer, out, t, chunks.append)
    assert s.decoded() == text
    if text.isascii():
        assert "".join(chunks) == text and all(chunks)


def _model_dir(tmp_path):
    cfg = Gpt2Config(vocab_size=VOCAB, n_positions=64, n_embd=36, n_layer=2, n_head=3, n_inner=100)
    w = synth.random_weights(cfg, 0x5EED0241, std=0.08, perturb=True)
    write_model_dir(tmp_path / "m", cfg, w)
    write_tokenizer(tmp_path / "m" / "tokenizer.json")
    return tmp_path / "m", cfg, w


@pytest.mark.gpu
def test_runtime_streams_text_of_the_tokens_the_oracle_generates(tmp_path):
    path, cfg, w = _model_dir(tmp_path)
    rt = Gpt2Runtime.from_dir(path)
    ref = oracle.Model(cfg, w)
    prompt = "hello there, quick fox"
    ids = rt.tokenizer.encode(prompt)
    want = ref.stream_token_ids_with_stats(ids, 20, None)[0]

    gen = TextGenerationConfig(max_new_tokens=20)
    seen = []
    tokens, st, prof = rt.stream_token_ids_with_stats(prompt, gen, seen.append)
    assert tokens == want and seen == want[len(ids):]
    assert st.prompt_tokens == len(ids) and st.generated_tokens == 20
    assert st.tokenize_time > 0.0 and prof.tokenization == st.tokenize_time

    chunks = []
    text, st2, prof2 = rt.stream_text_with_stats(prompt, gen, chunks.append)
    assert chunks[0] == prompt and len(chunks) == 21
    assert text == rt.tokenizer.decode(want)
    assert st2.generated_tokens == 20 and prof2.decoding > 0.0 and prof2.qkv_projection == 0.0
    text3, _, prof3 = rt.stream_text_with_stats(prompt, gen, lambda _t: None, profiled=True)
    assert text3 == text and prof3.qkv_projection > 0.0 and prof3.decoding > 0.0

    # greedy entry points: same tokens, no EOS rule
    assert rt.generate_greedy_text(prompt, 20) == text
    chunks = []
    assert rt.stream_greedy_text(prompt, 20, chunks.append) == text
    assert chunks[0] == prompt and len(chunks) == 21

    # the EOS id of the GPT-2 default (50256) lies outside this vocabulary
    with pytest.raises(Gpt2Error, match="is outside vocab_size 300") as e:
        rt.stream_greedy_text_with_stats(prompt, 4, lambda _t: None)
    assert e.value.kind == "InvalidConfig"
    # an EOS that the greedy run reaches ends the text before it
    eos = want[len(ids) + 5]
    first = want.index(eos, len(ids))
    text4, st4, _ = rt.stream_text_with_stats(prompt, TextGenerationConfig(20, eos_token_id=eos),
                                              lambda _t: None)
    assert st4.generated_tokens == first - len(ids)
    assert text4 == rt.tokenizer.decode(want[:first])


@pytest.mark.gpu
def test_runtime_from_dir_needs_the_tokenizer_file(tmp_path):
    path, _, _ = _model_dir(tmp_path)
    (path / "tokenizer.json").unlink()
    with pytest.raises(Gpt2Error, match="failed to load tokenizer"):
        Gpt2Runtime.from_dir(path)


def test_experiment_prompts_come_from_a_file_or_one_string(tmp_path):
    """load_experiment_prompts (src/main.rs:4009-4030)."""
    from puppygrad_amd import experiment as ex
    f = tmp_path / "prompts.txt"
    f.write_text("  first prompt \n\n\tsecond\n   \n")
    assert ex.load_experiment_prompts("ignored", str(f)) == ["first prompt", "second"]
    assert ex.load_experiment_prompts("only", None) == ["only"]
    f.write_text(" \n\n")
    with pytest.raises(ValueError, match="contains no prompts"):
        ex.load_experiment_prompts(None, str(f))
    with pytest.raises(ValueError, match="failed to read --prompt-file"):
        ex.load_experiment_prompts(None, str(tmp_path / "missing.txt"))
    with pytest.raises(ValueError, match="requires --prompt or --prompt-file"):
        ex.load_experiment_prompts(None, None)


@pytest.mark.gpu
def test_experiment_rows_over_text_prompts_carry_the_host_text_time(tmp_path):
    from puppygrad_amd import experiment as ex
    path, cfg, w = _model_dir(tmp_path)
    rt = Gpt2Runtime.from_dir(path)
    prompts = ["hello there, quick fox", "the lazy dog"]
    rows = ex.run_experiment(rt, prompts, [6], runs=2, warmup_runs=1, profile_runs=1,
                             eos_token_id=None)
    assert [r.prompt for r in rows] == prompts + ["<aggregate>"]
    assert [r.prompt_index for r in rows] == [0, 1, None]
    for r, p in zip(rows, prompts):
        assert r.prompt_tokens == len(rt.tokenizer.encode(p)) and r.generated_tokens == 6.0
        assert r.tokenize_ms > 0.0 and r.profile_tokenization_ms > 0.0 and r.profile_decoding_ms > 0.0
        assert r.profile_qkv_projection_ms > 0.0 and r.decode_ms > 0.0
    assert rows[2].runs == 4
    assert ex.format_csv(rows).count("\n") == 4
