"""
Command line of the framework:  python -m exllamav3_amd <command>

    models                                  the registered architectures
    generate --model DIR --tokens 1,2,3 [--tokens ...] [--max-new-tokens N] [--temperature T --top-k K --top-p P --seed S] [--dtype ...]
                                            token ids in, token ids out (one JSON line per prompt); prompts given together run as one batch
    trace --model DIR --dtype bfloat16|float32 --out DIR [--max-tokens N]
                                            replay steps from standard input and write logits (trace.py)

A model of the mixer family needs only libexl3_mix.so, which is compiled here on first use.
"""
from __future__ import annotations
import argparse
import json
import os
import shutil
import sys


def _dtype(name: str):
    import torch
    return {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}[name]


def _prepare(model_dir: str):
    """Compile what the model's architecture needs (and nothing else) before the GPU is touched."""
    from . import _lib, registry
    with open(os.path.join(model_dir, "config.json")) as f:
        arch = registry.architecture_of(json.load(f))
    if registry.native_libraries(arch) == ("mix",):
        hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
        if os.path.exists(hipcc) or shutil.which("hipcc"):
            try:
                _lib.ensure_mix_built()
            except Exception as e:               # e.g. a checkout that cannot be written: a library that is already there still serves
                if not os.path.exists(_lib.MIX_LIB_PATH):
                    raise
                print(f"exllamav3_amd: could not rebuild libexl3_mix.so ({type(e).__name__}: {e}); using the one that is there", file=sys.stderr)
        _lib.mixlib()
    else:
        _lib.lib()


def _load(args):
    import torch
    from . import registry
    if not torch.cuda.is_available():
        raise SystemExit("no GPU: the framework has no CPU path")
    _prepare(args.model)
    dt = _dtype(args.dtype)
    if dt == torch.float32:
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    return registry.load_model(args.model, "cuda:0", dt)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="exllamav3_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)
    sub.add_parser("models")
    g = sub.add_parser("generate")
    g.add_argument("--model", required=True)
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    g.add_argument("--tokens", action="append", required=True, help="comma-separated token ids of one prompt (repeat for a batch)")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=0)
    t = sub.add_parser("trace")
    t.add_argument("--model", required=True)
    t.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    t.add_argument("--out", required=True)
    t.add_argument("--max-tokens", type=int, default=0, help="most tokens alive at once: sizes the pages of a model whose cache grows with its sequences")
    args = ap.parse_args(argv)

    if args.cmd == "models":
        from . import registry
        print("\n".join(registry.architectures()))
        return 0
    if args.cmd == "generate":
        from .generator import Generator, SamplerSettings
        model = _load(args)
        prompts = [[int(x) for x in s.replace(" ", "").split(",") if x] for s in args.tokens]
        outs = Generator(model).generate(prompts, args.max_new_tokens, SamplerSettings(args.temperature, args.top_k, args.top_p, args.seed))
        for p, o in zip(prompts, outs):
            print(json.dumps({"prompt": p, "output": o}))
        return 0
    if args.cmd == "trace":
        from .trace import TraceSession
        os.makedirs(args.out, exist_ok=True)
        model = _load(args)
        TraceSession(model, args.out, args.max_tokens).run(sys.stdin)
        return 0
    return 2


if __name__ == "__main__":
    sys.exit(main())
