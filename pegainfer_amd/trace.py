"""Trace replay: feed given token ids through a model step by step and write the logits of the asked positions.

Reads one JSON object per line from standard input,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}
runs all entries of a step as ONE batch of the engine's step function (a request is admitted at its first entry and keeps
its cache between steps; "end" gives requests' pages and slots back), writes OUT/<step>.f32 ([wanted, vocab] little-endian
floats, in the order of the entries and of "want") for every step that asks for something, and prints "done <step>".
Nothing is sampled.  The engine comes from the model registry; its cache holds --max-tokens tokens and four requests.
"""
import argparse
import json
import os
import sys


def main(argv=None):
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, default=4096, help="cache capacity in tokens")
    ap.add_argument("--max-requests", type=int, default=4, help="request slots")
    a = ap.parse_args(argv)

    from . import registry
    cfg = registry.read_config(a.model)
    fam = registry.family_of(cfg)
    if fam is None:
        print("no engine is registered for this model", file=sys.stderr)
        return 2
    if a.dtype not in registry.REGISTRY[fam][1]:
        print("%s is not served in %s" % (fam, a.dtype), file=sys.stderr)
        return 3
    eng = registry.load_engine(a.model, dtype=a.dtype, max_tokens=a.max_tokens, max_requests=a.max_requests)
    if not hasattr(eng, "step"):
        print("the %s engine has no batched step over portions" % fam, file=sys.stderr)
        return 2
    os.makedirs(a.out, exist_ok=True)
    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries, want, off = [], [], 0
        for e in st["entries"]:
            if e["id"] not in live:
                live[e["id"]] = eng.new_request()
            entries.append((live[e["id"]], e["tokens"]))
            want += [off + int(w) for w in e.get("want", [])]
            off += len(e["tokens"])
        if entries:
            lg = eng.step(entries, want=want, logits=True)
            if want:
                tmp = os.path.join(a.out, ".%s.part" % st["step"])
                with open(tmp, "wb") as f:
                    f.write(lg.astype("<f4").tobytes())
                os.replace(tmp, os.path.join(a.out, "%s.f32" % st["step"]))
        for rid in st.get("end", []):
            if rid in live:
                eng.drop_request(live.pop(rid))
        sys.stdout.write("done %s\n" % st["step"])
        sys.stdout.flush()
    eng.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
