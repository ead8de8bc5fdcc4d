"""Command line: generate from a model folder (or a configuration with random weights).

In the manner of the reference's launcher (``scripts/gesso-serve.jl:62-84``): flags take a value,
except ``--cpu`` and ``--check``; an unknown flag is an error, because a mistyped flag silently
ignored would run the wrong thing.  ``--model`` stands where the reference has ``--gguf``,
``--n-ctx`` is the context length, ``--model-id`` a name that is echoed in the output,
``--check`` a self-test on a tiny random model that needs no files, ``--cpu`` is refused: this
engine has no CPU path.  The server's ``--host``/``--port`` have no counterpart: no server here.

    python -m gesso_amd --model DIR --prompt-ids 1,2,3 --max-new-tokens 16
    python -m gesso_amd --config config.json --random-weights 0 --prompt-ids 5,6 --temperature 0.8 --seed 7
    python -m gesso_amd --check
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import List


def parse_launch(argv: List[str]) -> argparse.Namespace:
    ap = argparse.ArgumentParser(prog="gesso_amd", description="LFM2 generation on one MI355X", allow_abbrev=False)
    ap.add_argument("--model", help="folder with config.json and model.safetensors")
    ap.add_argument("--config", help="a config.json alone; needs --random-weights")
    ap.add_argument("--random-weights", type=int, metavar="SEED", help="draw weights from this seed")
    ap.add_argument("--n-ctx", type=int, default=None, help="context length: most tokens a request may hold")
    ap.add_argument("--model-id", default=None, help="a name for the model, echoed in the output")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prompt-ids", action="append", default=[], metavar="1,2,3",
                    help="a prompt as comma-separated token ids; may be given several times")
    ap.add_argument("--prompt-file", help="a file with one prompt per line, ids separated by commas or blanks")
    ap.add_argument("--max-new-tokens", type=int, default=8)
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--eos-id", type=int, action="append", default=None, help="stop at this id (default: the configuration's)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--prefill-chunk", type=int, default=None, help="largest portion of a prompt per step (GESSO_PREFILL_CHUNK)")
    ap.add_argument("--max-num-seqs", type=int, default=64)
    ap.add_argument("--gemm", default="auto", choices=["auto", "own", "library"],
                    help="products of more than 64 rows: the vendor library where it is faster (auto), the hand-written "
                         "kernel everywhere (own), the library wherever it can go (library)")
    ap.add_argument("--record-portions", action="store_true",
                    help="steps with prompt portions whose kind recurs are recorded as HIP graphs and replayed (pays where "
                         "the host's launches, not the kernels, bound such a step: small models, small portions)")
    ap.add_argument("--poison", action="store_true", help="debugging: fill pages and slots that are given back with NaN")
    ap.add_argument("--cpu", action="store_true", help="refused: there is no CPU path")
    ap.add_argument("--check", action="store_true", help="self-test on a tiny random model")
    return ap.parse_args(argv)


def _ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def run_check() -> int:
    from .config import Lfm2Config
    from .engine.session import Session

    cfg = Lfm2Config(vocab_size=64, hidden_size=32, num_hidden_layers=2, num_attention_heads=2,
                     num_key_value_heads=1, layer_types=("conv", "full_attention"), conv_L_cache=3, conv_bias=False,
                     intermediate_size=48, norm_eps=1e-5, rope_theta=1e4, tie_word_embeddings=True,
                     max_position_embeddings=64)
    s = Session(cfg, random_weights_seed=0, random_weights_std=0.1, dtype="float32", context_length=32)
    a = s.generate([1, 2, 3], max_new_tokens=4)
    b = s.generate([1, 2, 3], max_new_tokens=4)
    if a != b or len(a) != 7:
        print("gesso_amd check failed: generation is not reproducible", file=sys.stderr)
        return 1
    print("gesso_amd check ok (tiny random model, 4 tokens, twice the same)")
    return 0


def main(argv=None) -> int:
    args = parse_launch(sys.argv[1:] if argv is None else argv)
    if args.cpu:
        print("gesso_amd: --cpu is refused: the engine runs on the GPU only", file=sys.stderr)
        return 2
    if args.check:
        return run_check()
    if (args.model is None) == (args.config is None):
        print("gesso_amd: give --model DIR, or --config FILE with --random-weights SEED", file=sys.stderr)
        return 2
    prompts = [_ids(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [_ids(line) for line in f if line.strip()]
    if not prompts:
        print("gesso_amd: no prompt given (--prompt-ids or --prompt-file)", file=sys.stderr)
        return 2

    from .engine.session import Session
    from .parts.runtime import RuntimeOptions

    kw = dict(dtype=args.dtype, page_size=args.page_size, context_length=args.n_ctx, chunk_size=args.prefill_chunk,
              max_num_seqs=args.max_num_seqs, kernel_options=RuntimeOptions(many_rows=args.gemm, record_portions=args.record_portions),
              poison=args.poison)
    if args.model is not None:
        session = Session(args.model, **kw)
    else:
        if args.random_weights is None:
            print("gesso_amd: --config needs --random-weights SEED", file=sys.stderr)
            return 2
        from .config.jsonio import load_strict
        from .config.registry import architecture_of
        raw = load_strict(args.config)
        session = Session(architecture_of(raw).parse(raw), random_weights_seed=args.random_weights, **kw)
    out = session.generate(prompts, max_new_tokens=args.max_new_tokens, temperature=args.temperature,
                           top_p=args.top_p, seed=args.seed, eos_ids=args.eos_id)
    st = session.last_stats
    print(json.dumps({"model": args.model_id or args.model or args.config, "dtype": args.dtype,
                      "ids": out, "new_tokens": st.get("new_tokens"), "prefill_ms": round(st.get("prefill_ms", 0), 3),
                      "decode_ms": round(st.get("decode_ms", 0), 3), "steps": st.get("steps"),
                      "preemptions": st.get("preemptions")}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
