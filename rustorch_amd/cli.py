"""`python -m rustorch_amd.cli --model m.gguf --tokenizer tokenizer.json --prompt "..."`: the generation path of
the reference CLI (example-cli/src/model/inference.rs:91-211, cli/args.rs:69-141 with `--backend hip`) on this
backend: GGUF file -> device model, prompt -> ids, prefill, decode loop with sampling, ids -> text, and the
metrics the reference prints (time to first token, tokens/s)."""
from __future__ import annotations

import argparse
import json
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="rustorch_amd.cli", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="llama-architecture GGUF file")
    ap.add_argument("--tokenizer", help="Hugging Face tokenizer.json; without it --prompt-ids is required and ids are printed")
    ap.add_argument("--prompt", help="prompt text")
    ap.add_argument("--prompt-ids", help="comma-separated token ids instead of text")
    ap.add_argument("--backend", default="hip", choices=["hip"], help="only the MI355X backend exists here")
    ap.add_argument("--device", type=int, default=0)
    ap.add_argument("--max-tokens", type=int, default=64)
    ap.add_argument("--max-context", type=int, default=None, help="positions to reserve in the cache (default: the file's context length)")
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--repetition-penalty", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--json", action="store_true", help="print the metrics as one JSON line")
    args = ap.parse_args(argv)

    import numpy as np
    from . import llama
    from .executor import HipKernelExecutor
    from .metrics import InferenceTimer, MetricsCollector
    from .sampling import SamplingConfig
    from .tokenizer import TokenizerWrapper

    tok = TokenizerWrapper.from_file(args.tokenizer) if args.tokenizer else None
    if args.prompt_ids:
        ids = [int(v) for v in args.prompt_ids.split(",") if v.strip()]
    elif args.prompt is not None and tok is not None:
        ids = tok.encode(args.prompt, True)
    else:
        ap.error("give --prompt with --tokenizer, or --prompt-ids")
    if not ids:
        ap.error("the prompt is empty")
    if args.temperature <= 0:
        cfg = SamplingConfig.greedy()
    else:
        cfg = SamplingConfig(temperature=args.temperature, top_k=args.top_k or None, top_p=args.top_p if args.top_p < 1.0 else None,
                             repetition_penalty=args.repetition_penalty)
    import os
    with HipKernelExecutor(args.device) as ex:
        need = len(ids) + args.max_tokens
        model = llama.load_gguf(ex, args.model, max_pos=max(need, args.max_context or 0) or None)
        try:
            timer = InferenceTimer()
            timer.start()
            out = []

            def on_token(t):
                timer.mark_first_token()
                timer.mark_token()
                out.append(int(t))

            eos = tok.eos_token_id() if tok else None
            llama.generate(model, ids, args.max_tokens, cfg, eos_token=eos, rng=np.random.default_rng(args.seed), on_token=on_token)
            timer.end()
        finally:
            model.close()
        m = MetricsCollector()
        m.set_backend("hip:%d" % args.device)
        m.set_model_size(os.path.getsize(args.model))
        if timer.ttft_ms() is not None:
            m.set_ttft(timer.ttft_ms())
        if timer.tokens_per_sec() is not None:
            m.set_tokens_per_sec(timer.tokens_per_sec())
        m.set_total_time(timer.total_ms() or 0.0)
    text = tok.decode(out, True) if tok else ",".join(str(t) for t in out)
    print(text)
    if args.json:
        print(json.dumps({"backend": m.backend, "prompt_tokens": len(ids), "generated_tokens": len(out), "ttft_ms": m.ttft,
                          "total_ms": m.total_time, "tokens_per_sec": m.tokens_per_sec, "model_bytes": m.model_size,
                          "meets_ttft_target": m.meets_ttft_target(), "meets_tps_target": m.meets_tps_target()}), file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
