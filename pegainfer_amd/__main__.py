"""Command line of the package:  python -m pegainfer_amd <command> ...

  generate   greedy / sampled generation of token ids through the continuous-batching scheduler
  trace      replay a trace of token ids step by step and write the asked logits (same program as bin/trace_run)
  build      compile the native libraries (same as python -m pegainfer_amd.build)
  models     list the registered model families and the dtypes they are served in

The model family is read from the folder's config.json (pegainfer_amd/registry.py).  Token ids in, token ids out: the
tokenizer lives outside this package.
"""
import argparse
import json
import sys


def _generate(a):
    from . import registry
    from . import scheduler as S
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt_ids]
    if a.prompt_file:
        with open(a.prompt_file) as f:
            prompts += [json.loads(line) for line in f if line.strip()]
    if not prompts:
        raise SystemExit("no prompt: give --prompt-ids 1,2,3 (repeatable) or --prompt-file with one JSON list per line")
    need = sum(-(-(len(p) + a.max_new_tokens) // 16) * 16 for p in prompts)
    eng = registry.load_engine(a.model, dtype=a.dtype, max_tokens=max(a.max_tokens, need), max_requests=max(len(prompts), 1))
    sch = registry.scheduler_for(eng, seed=a.seed, stop_tokens=a.stop_token)
    params = (a.temperature, a.top_k, a.top_p, not a.stop_token)
    rids = [sch.submit(p, a.max_new_tokens, params=params) for p in prompts]
    out = {r: [] for r in rids}
    while True:
        plan = sch.step()
        for ev in sch.poll():
            if ev[1] == S.TOKEN:
                out[ev[0]].append(int(ev[2]))
            elif ev[1] in (S.ERROR, S.REJECTED):
                raise SystemExit("request %d failed: %s" % (ev[0], sch.last_message()))
        if plan <= 0 and sch.num_active() == 0 and sch.num_deferred() == 0:
            break
    for r, p in zip(rids, prompts):
        print(json.dumps({"prompt": p, "tokens": out[r]}))
    sch.close()
    eng.close()
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m pegainfer_amd", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate", help="generate token ids for one or more prompts")
    g.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    g.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; repeat for several requests")
    g.add_argument("--prompt-file", help="one JSON list of token ids per line")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--max-tokens", type=int, default=4096, help="cache capacity in tokens")
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-k", type=int, default=-1)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=42)
    g.add_argument("--stop-token", type=int, action="append", default=[])
    t = sub.add_parser("trace", help="replay a trace from standard input (see pegainfer_amd/trace.py)", add_help=False)
    t.add_argument("rest", nargs=argparse.REMAINDER)
    sub.add_parser("build", help="compile the native libraries")
    sub.add_parser("models", help="list the registered model families")
    a = ap.parse_args(argv)
    if a.cmd == "generate":
        return _generate(a)
    if a.cmd == "trace":
        from .trace import main as trace_main
        return trace_main(a.rest)
    if a.cmd == "build":
        from . import build
        build.build(verbose=True)
        return 0
    from . import registry
    for fam, (_, dtypes) in registry.REGISTRY.items():
        print("%-10s %s" % (fam, ", ".join(dtypes)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
