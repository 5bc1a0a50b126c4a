"""Randomised parity of the HIP sampler with the CPU oracle over shapes, element types, parameters
and row structures the fixed tests do not enumerate.

    python tests/fuzz_parity.py --cases 2000 --seed 1

Every case draws a vocabulary size (1 .. 300 000, biased to small and to sizes around the
vectorisation and LDS limits), an element type, a row pitch (aligned or not), a temperature, top-p,
top-k and a row structure (normal, peaked, few distinct values, flat, wide range, tiny magnitudes,
masked with -inf, sorted), samples a few rows on the device with and without debug records and
compares tokens, coin states and the softmax normaliser (bit for bit) with the oracle (test infrastructure, never the thing measured) in
the arithmetic the HIP sampler implements.  Prints one JSON line; exits non-zero on a mismatch and
names the case.  Not collected by pytest.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def make_rows(rng, kind, rows, vocab):
    x = rng.standard_normal((rows, vocab)).astype(np.float32)
    if kind == "normal":
        x *= np.float32(rng.choice([0.3, 1.0, 2.0, 5.0]))
    elif kind == "peaked":
        for b in range(rows):
            hot = rng.integers(0, vocab, size=min(vocab, int(rng.integers(1, 30))))
            x[b, hot] += np.float32(rng.choice([4.0, 8.0, 15.0]))
    elif kind == "few":
        k = int(rng.integers(1, 40))
        vals = (rng.standard_normal(k) * 3.0).astype(np.float32)
        x = vals[rng.integers(0, k, size=(rows, vocab))]
    elif kind == "flat":
        x = np.full((rows, vocab), np.float32(rng.standard_normal()), dtype=np.float32)
    elif kind == "wide":
        x *= np.float32(40.0)
    elif kind == "tiny":
        x *= np.float32(1e-30)
    elif kind == "masked":
        x[rng.random((rows, vocab)) < rng.choice([0.3, 0.9, 0.999])] = -np.inf
    elif kind == "sorted":
        x = np.sort(x, axis=1)
        if rng.random() < 0.5:
            x = x[:, ::-1]
    return np.ascontiguousarray(x)


def run(cases=2000, seed=1, max_vocab=300000, configs=False):
    """The cases; returns {"cases", "failures", "first_failures", "seconds"}."""
    args = argparse.Namespace(cases=cases, seed=seed, max_vocab=max_vocab, configs=configs)

    import torch

    import executorch_amd as ea
    from executorch_amd import workloads as W
    from oracle import oracle as O
    from util import to_device

    O.build()
    assert torch.cuda.is_available(), "fuzz_parity.py needs a GPU"
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(args.seed)
    special = [1, 2, 3, 7, 8, 63, 64, 65, 1023, 1024, 1025, 4095, 4096, 4097, 8191, 8192, 8200, 16383, 16384, 16385, 16400,
               32000, 32768, 65536, 128256, 131072, 151936, 262144]
    kinds = ["normal", "peaked", "few", "flat", "wide", "tiny", "masked", "sorted"]
    dtypes = [W.DTYPE_FLOAT, W.DTYPE_HALF, W.DTYPE_BFLOAT16]
    failures = []
    t0 = time.time()
    for case in range(args.cases):
        r = rng.random()
        if r < 0.35:
            vocab = int(rng.choice(special))
        elif r < 0.8:
            vocab = int(rng.integers(1, 20000))
        else:
            vocab = int(rng.integers(20000, args.max_vocab))
        vocab = min(vocab, args.max_vocab)
        dtype = int(rng.choice(dtypes))
        kind = str(rng.choice(kinds))
        rows = int(rng.integers(1, 9 if args.configs else 5))
        if args.configs and rng.random() < 0.05:
            # now and then enough rows for the groups of a call to share the compute units unevenly
            rows = int(rng.integers(9, 41))
        temperature = float(rng.choice([0.05, 0.3, 0.6, 0.8, 1.0, 1.5, 7.0, 50.0, -1.0, 0.0]))
        topp = float(rng.choice([0.0, 0.02, 0.5, 0.8, 0.9, 0.95, 0.999, 1.0]))
        topk = int(rng.choice([0, 0, 0, 1, 2, 40, 64, 65, 256, 257, 1000, vocab - 1, vocab, vocab + 5]))
        pad = int(rng.choice([0, 0, 1, 3, 8]))
        seed = int(rng.integers(0, 2**31))
        label = dict(case=case, vocab=vocab, dtype=W.DTYPE_NAMES[dtype], kind=kind, rows=rows, temperature=temperature,
                     topp=topp, topk=topk, pad=pad, seed=seed)
        xf = make_rows(rng, kind, rows, vocab)
        x = W.to_storage(xf, dtype)
        padded = np.zeros((rows, vocab + pad), dtype=x.dtype)
        padded[:, :vocab] = x
        dx = to_device(padded, dtype, dev)[:, :vocab]  # row pitch vocab + pad elements
        states = (np.uint64(seed) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
        try:
            if args.configs:
                cfgs = []
                want = np.empty(rows, dtype=np.int32)
                for b in range(rows):
                    t_b = float(rng.choice([0.05, 0.6, 1.0, 7.0, 0.0, -1.0]))  # -1: the sampler's own
                    p_b = float(rng.choice([0.0, 0.5, 0.9, 0.999, 1.0]))
                    k_b = int(rng.choice([0, 0, 1, 40, 257, vocab - 1, vocab + 1]))
                    seed_b = int(rng.choice([0, int(rng.integers(1, 2**31))]))  # 0: continue the row's stream
                    cfgs.append((t_b, p_b, k_b, seed_b))
                    st_b = np.array([seed_b if seed_b else states[b]], dtype=np.uint64)
                    t_eff = max(temperature, 0.0) if t_b < 0 else t_b
                    want[b] = O.sample_rows(np.ascontiguousarray(x[b:b + 1]), dtype, O.inv_temperature(t_eff), p_b, k_b, st_b,
                                            mode=O.MODE_UPCAST, tie=O.TIE_STABLE)[0][0]
                    states[b] = st_b[0]
                label["configs"] = cfgs
                s = ea.Sampler(vocab, max(temperature, 0.0), topp, seed, max_batch=rows)
                got = s.sample_batch_configs(dx, cfgs).cpu().numpy()
                after = s.get_rng_states(rows)
                got_plain = got
                ok = np.array_equal(got, want) and np.array_equal(after, states)
            else:
                s = ea.Sampler(vocab, temperature, topp, seed, max_batch=rows)
                s.set_topk(topk)
                ddbg = torch.zeros((rows, 8), dtype=torch.int32, device=dev)
                got = s.sample_batch(dx, debug_out=ddbg).cpu().numpy()
                after = s.get_rng_states(rows)
                plain = ea.Sampler(vocab, temperature, topp, seed, max_batch=rows)
                plain.set_topk(topk)
                got_plain = plain.sample_batch(dx).cpu().numpy()
                # the constructor does not clamp: a negative temperature gives a negative inverse (sampler.cpp:173-181)
                want, ex = O.sample_rows(np.ascontiguousarray(x), dtype, O.inv_temperature(temperature), topp, topk, states,
                                         mode=O.MODE_UPCAST, tie=O.TIE_STABLE, threads=4, explain=True)
                ok = np.array_equal(got, want) and np.array_equal(got_plain, want) and np.array_equal(after, states)
                if temperature != 0.0:  # the softmax normaliser, bit for bit (the arg-max computes none)
                    sums = ea.debug_records(ddbg)["sum"]
                    for b in range(rows):
                        a, w_ = np.float32(sums[b]), np.float32(ex[b].sum)
                        if not (a.view(np.uint32) == w_.view(np.uint32) or (np.isnan(a) and np.isnan(w_))):
                            ok = False
                            label["sum"] = [b, float(a), float(w_)]
        except Exception as e:  # an error status is a failure here: every case is a legal call
            ok = False
            label["error"] = repr(e)[:300]
            got = want = got_plain = None
        if not ok:
            label.update(got=None if got is None else got.tolist(), want=None if want is None else want.tolist(),
                         got_plain=None if got_plain is None else got_plain.tolist())
            failures.append(label)
            print("fuzz_parity: MISMATCH", json.dumps(label), file=sys.stderr, flush=True)
            if len(failures) >= 10:
                break
        if case % 100 == 99:
            print(f"fuzz_parity: {case + 1} cases, {len(failures)} failures, {time.time() - t0:.0f} s", file=sys.stderr, flush=True)
    return {"cases": case + 1, "failures": len(failures), "first_failures": failures[:3], "seconds": round(time.time() - t0, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--cases", type=int, default=2000)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--max-vocab", type=int, default=300000)
    ap.add_argument("--configs", action="store_true",
                    help="give every row its own (temperature, top-p, top-k, seed) through sample_batch_configs")
    args = ap.parse_args()
    res = run(args.cases, args.seed, args.max_vocab, args.configs)
    print(json.dumps(res))
    sys.exit(1 if res["failures"] else 0)


if __name__ == "__main__":
    main()
