"""Tokenizer wrapper and timing objects of the CLI (example-cli/src/tokenizer/wrapper.rs, metrics/timing.rs,
metrics/mod.rs) and, on the GPU, the command line from a GGUF file and a tokenizer file to text."""
import json
import time

import numpy as np
import pytest


def tiny_tokenizer_file(path, vocab_size):
    """A word-level tokenizer.json with <s>, </s>, <unk> and w0..wN, written with the tokenizers library itself."""
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    vocab = {"<unk>": 0, "<s>": 1, "</s>": 2}
    for i in range(3, vocab_size):
        vocab["w%d" % i] = i
    t = Tokenizer(WordLevel(vocab, unk_token="<unk>"))
    t.pre_tokenizer = Whitespace()
    t.save(str(path))


def test_tokenizer_wrapper(tmp_path):
    from rustorch_amd.tokenizer import TokenizerWrapper
    from rustorch_amd.errors import InvalidParameters
    d = TokenizerWrapper.dummy()                      # wrapper.rs:108-131: the dummy answers without panicking
    assert isinstance(d.encode("test", False), list)
    assert d.bos_token_id() is None and d.eos_token_id() is None and d.pad_token_id() is None and d.unk_token_id() is None
    with pytest.raises(InvalidParameters, match="not found"):
        TokenizerWrapper.from_file(tmp_path / "missing.json")
    bad = tmp_path / "bad.json"
    bad.write_text("{ not a tokenizer")
    with pytest.raises(InvalidParameters, match="Failed to load"):
        TokenizerWrapper.from_file(bad)
    p = tmp_path / "tokenizer.json"
    tiny_tokenizer_file(p, 50)
    t = TokenizerWrapper.from_file(p)
    assert t.vocab_size() == 50
    assert t.bos_token_id() == 1 and t.eos_token_id() == 2 and t.unk_token_id() == 0 and t.pad_token_id() is None
    ids = t.encode("w5 w7 nope w49", False)
    assert ids == [5, 7, 0, 49]
    assert t.decode([5, 7, 49], True) == "w5 w7 w49"


def test_inference_timer_and_targets():
    from rustorch_amd.metrics import InferenceTimer, MetricsCollector
    t = InferenceTimer()
    assert t.ttft_ms() is None and t.tokens_per_sec() is None and t.avg_token_time_ms() is None
    t.mark_token()                                    # before start: ignored (timing.rs:153-157)
    assert t.token_times == []
    t.start()
    time.sleep(0.01)
    t.mark_first_token(); t.mark_token()
    first = t.ttft
    time.sleep(0.005)
    t.mark_first_token(); t.mark_token()              # only the first call sets the time to first token
    t.end()
    assert t.ttft == first and 8.0 <= t.ttft_ms() <= 200.0
    assert len(t.token_times) == 2 and t.total_ms() >= t.ttft_ms()
    assert abs(t.tokens_per_sec() - 2 / t.total_time) < 1e-9
    m = MetricsCollector()
    assert not m.meets_all_targets()
    m.set_ttft(150.0); m.set_tokens_per_sec(25.0); m.set_model_size(1000); m.set_memory_usage(1400)
    assert m.meets_ttft_target() and m.meets_tps_target() and m.meets_memory_target() and m.meets_all_targets()
    assert abs(m.memory_efficiency() - 1000 / 1400) < 1e-12
    m.set_ttft(200.0)                                 # strict comparisons (mod.rs:93-100)
    assert not m.meets_ttft_target()
    m.set_tokens_per_sec(20.0)
    assert not m.meets_tps_target()
    m.set_memory_usage(1500)
    assert not m.meets_memory_target()


@pytest.mark.gpu
def test_cli_from_files_to_text(ex, tmp_path, capsys):
    """GGUF file + tokenizer file + prompt -> text: the same ids as driving the model object directly."""
    from rustorch_amd import cli, llama
    from rustorch_amd.tokenizer import TokenizerWrapper
    cfg = dict(n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=128)
    model_path, tok_path = tmp_path / "m.gguf", tmp_path / "tokenizer.json"
    llama.write_synthetic_gguf(model_path, 43, context=64, **cfg)
    tiny_tokenizer_file(tok_path, cfg["vocab"])
    prompt = "w5 w17 w99 w3 w64"
    rc = cli.main(["--model", str(model_path), "--tokenizer", str(tok_path), "--prompt", prompt, "--max-tokens", "9", "--json"])
    assert rc == 0
    cap = capsys.readouterr()
    text = cap.out.strip().splitlines()[-1]
    metrics = json.loads(cap.err.strip().splitlines()[-1])
    tok = TokenizerWrapper.from_file(tok_path)
    ids = tok.encode(prompt, True)
    gm = llama.load_gguf(ex, model_path, max_pos=64)
    want = llama.generate(gm, ids, 9, eos_token=tok.eos_token_id())
    gm.close()
    assert text == tok.decode(want, True)
    assert metrics["prompt_tokens"] == len(ids) and metrics["generated_tokens"] == len(want)
    assert metrics["ttft_ms"] > 0 and metrics["total_ms"] >= metrics["ttft_ms"] and metrics["tokens_per_sec"] > 0
    # ids in, ids out without a tokenizer; sampling flags reach the sampler
    rc = cli.main(["--model", str(model_path), "--prompt-ids", "5,17,99", "--max-tokens", "4", "--temperature", "0.8", "--top-k", "5", "--seed", "3"])
    assert rc == 0
    out_ids = [int(v) for v in capsys.readouterr().out.strip().splitlines()[-1].split(",")]
    assert len(out_ids) == 4 and all(0 <= v < cfg["vocab"] for v in out_ids)
