"""Randomised parity of the device-side logit processor chain with its CPU restatement.

    python tests/fuzz_logit_chain.py --cases 1000 --seed 1

Every case draws a tensor (rank 2 or 3, 1..6 rows, a vocabulary that is small, near the 8192-entry
tile boundaries or up to 200 000, one of three element types, values with zeros, infinities, NaN
and numbers near the 16-bit types' limits) and a chain of 1..8 processors with random parameters:
bias, scale, mask and per-token bias lists with duplicate and out-of-range ids, repetition
penalties over histories with repeats, out-of-range ids and zero lengths.  The chain runs once on
the device and the restatement (test infrastructure, never the thing measured) processor by
processor on the host; every element must be equal bit for bit (NaN with NaN), and the sequence
positions before the last one of a rank-3 tensor must be untouched.  Prints one JSON line; exits
non-zero on a mismatch and names the case.  tests/test_gpu_logit_processor.py runs a few hundred
cases of it with every GPU suite.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def make_values(rng, shape, kind, lpo):
    x = (rng.standard_normal(shape) * np.float32(rng.choice([0.5, 3.0, 30.0]))).astype(np.float32)
    flat = x.reshape(-1)
    n = flat.size
    specials = [0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, -65504.0, 6e-8, 1e-38, 3e38, -3e38, 1.0, -1.0]
    for v in specials:
        if rng.random() < 0.5:
            flat[rng.integers(0, n, size=max(1, n // 500))] = np.float32(v)
    return lpo.storage_round(x, kind)


def run(cases=1000, seed=1, max_vocab=200000, stop_after=10):
    """The comparison; returns the report as a dict (stops after `stop_after` mismatches)."""
    args = argparse.Namespace(cases=cases, seed=seed, max_vocab=max_vocab)

    import torch

    from executorch_amd.logit_processor import LogitChain
    from oracle import logit_processor_oracle as lpo

    assert torch.cuda.is_available(), "fuzz_logit_chain.py needs a GPU"
    dev = torch.device("cuda:0")
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
    rng = np.random.default_rng(args.seed)
    special = [1, 2, 63, 64, 65, 255, 256, 257, 8191, 8192, 8193, 16383, 16384, 16385, 24576, 32000, 65536, 128256]
    failures = []
    t0 = time.time()
    for case in range(args.cases):
        r = rng.random()
        if r < 0.4:
            vocab = int(rng.choice(special))
        elif r < 0.85:
            vocab = int(rng.integers(1, 20000))
        else:
            vocab = int(rng.integers(20000, args.max_vocab))
        vocab = min(vocab, args.max_vocab)
        kind = str(rng.choice(["f32", "f16", "bf16"]))
        batch = int(rng.integers(1, 7))
        rank = int(rng.choice([2, 3]))
        shape = (batch, vocab) if rank == 2 else (batch, int(rng.integers(1, 4)), vocab)
        x = make_values(rng, shape, kind, lpo)
        hist_len = int(rng.choice([1, 5, 64, 300, 1500]))
        history = rng.integers(-3, vocab + 3, size=(batch, hist_len)).astype(np.int32)
        if hist_len >= 64:
            history[:, 10:30] = history[:, 40:60]  # repeats inside a row's history
        lengths = rng.integers(0, hist_len + 1, size=batch).astype(np.int32)
        if rng.random() < 0.3:
            lengths[int(rng.integers(0, batch))] = hist_len
        d_hist, d_len = torch.from_numpy(history).to(dev), torch.from_numpy(lengths).to(dev)

        recipe = []
        want = x.copy()
        chain = LogitChain()
        label = dict(case=case, shape=list(shape), kind=kind, hist_len=hist_len)
        try:
            for _ in range(int(rng.integers(1, 9))):
                op = str(rng.choice(["bias", "scale", "mask", "tb", "rep"]))
                if op == "bias":
                    v = float(rng.choice([0.0, -1.25, 0.1, 1e-3, 100.0, -7.5, 70000.0]))
                    chain.add_bias(v); lpo.add_bias(want, v, kind); recipe.append((op, v))
                elif op == "scale":
                    v = float(rng.choice([1.0, 0.7, -1.5, 1.0 / 3.0, 0.0, 1e-4, 300.0]))
                    chain.add_scale(v); lpo.scale(want, v, kind); recipe.append((op, v))
                elif op == "mask":
                    ids = rng.integers(-2, vocab + 2, size=int(rng.choice([1, 3, 17, 200]))).astype(np.int32)
                    chain.add_mask(ids); lpo.mask(want, ids, kind); recipe.append((op, ids.size))
                elif op == "tb":
                    n = int(rng.choice([1, 4, 33, 257]))
                    ids = rng.integers(-2, vocab + 2, size=n).astype(np.int32)
                    if n >= 4:
                        ids[n // 2:] = ids[:n - n // 2]  # every id of the first half listed twice
                    val = (rng.standard_normal(n) * np.float32(rng.choice([0.01, 2.0, 50.0]))).astype(np.float32)
                    chain.add_token_bias(ids, val); lpo.token_bias(want, ids, val, kind); recipe.append((op, n))
                else:
                    v = float(rng.choice([1.0, 1.3, 0.8, 1.7, 5.0, 1e-3]))
                    chain.add_repetition_penalty(v, d_hist, d_len)
                    lpo.repetition_penalty(want, v, history, lengths, kind)
                    recipe.append((op, v))
            label["recipe"] = recipe
            t = torch.from_numpy(x).to(dev).to(tdt[kind]).contiguous()
            chain.process(t)
            got = t.float().cpu().numpy()
            same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
            ok = bool(same.all())
            if not ok:
                where = np.argwhere(~same)[:5]
                label.update(where=where.tolist(), got=[repr(float(v)) for v in got[~same][:5]],
                             want=[repr(float(v)) for v in want[~same][:5]], start=[repr(float(v)) for v in x[~same][:5]])
            chain.close()
        except Exception as e:  # an error status is a failure here: every case is a legal call
            ok = False
            label["recipe"] = recipe
            label["error"] = repr(e)[:300]
        if not ok:
            failures.append(label)
            print("fuzz_logit_chain: MISMATCH", json.dumps(label), file=sys.stderr, flush=True)
            if len(failures) >= stop_after:
                break
        if case % 100 == 99:
            print(f"fuzz_logit_chain: {case + 1} cases, {len(failures)} failures, {time.time() - t0:.0f} s", file=sys.stderr,
                  flush=True)
    return {"cases": case + 1, "failures": len(failures), "first_failures": failures[:3], "seconds": round(time.time() - t0, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--cases", type=int, default=1000)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--max-vocab", type=int, default=200000)
    args = ap.parse_args()
    res = run(args.cases, args.seed, args.max_vocab)
    print(json.dumps(res))
    sys.exit(1 if res["failures"] else 0)


if __name__ == "__main__":
    main()
