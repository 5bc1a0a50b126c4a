"""Parity of the HIP sampler with the CPU oracle over many seeded rows of one workload.

    python tests/parity_report.py --workload cfg2 --rows 100000

Rows of the workload's distribution are generated on the device in chunks, sampled there, copied
to the host and sampled by the oracle (test infrastructure, never the thing measured):

  * against the oracle in the arithmetic the HIP sampler implements (rows converted to fp32, exactly
    tied probabilities ordered by token index): every token must be equal;
  * against the same arithmetic with the reference's own tie order (what std::sort leaves): rows that
    differ are counted, and each must carry equal probabilities on the two tokens;
  * against the reference's native 16-bit arithmetic (sample<BFloat16> / sample<Half>): agreement is
    counted and reported, not required (every intermediate is rounded to 8 / 11 bits there).

Prints one JSON line.  tests/test_gpu_parity_sweep.py runs the same function inside the GPU suite
(100 000 rows of cfg2, a few thousand of the other workloads).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def device_rows(w, rows, gen, torch, dev):
    """[rows, vocab] of the workload's distribution in its storage type, made on the device."""
    from executorch_amd import workloads as W

    tdt = {W.DTYPE_FLOAT: torch.float32, W.DTYPE_HALF: torch.float16, W.DTYPE_BFLOAT16: torch.bfloat16}[w.dtype]
    x = torch.randn((rows, w.vocab), generator=gen, device=dev, dtype=torch.float32)
    if w.kind == "normal2":
        x *= 2.0
    elif w.kind == "normal15":
        x *= 1.5
    elif w.kind == "flat":
        x *= 0.5
    elif w.kind == "peaked":
        ids = torch.rand((rows, w.vocab), generator=gen, device=dev).topk(20, dim=1).indices  # 20 distinct ids per row
        x.scatter_add_(1, ids, torch.full(ids.shape, 8.0, device=dev))
    elif w.kind == "mixed":  # odd rows: Gumbel(0, 1) noise and one id raised by 12
        odd = torch.arange(1, rows, 2, device=dev)
        u = torch.rand((odd.numel(), w.vocab), generator=gen, device=dev).clamp_(1e-7, 1.0 - 1e-7)
        g = -torch.log(-torch.log(u))
        hot = torch.randint(0, w.vocab, (odd.numel(),), generator=gen, device=dev)
        g[torch.arange(odd.numel(), device=dev), hot] += 12.0
        x[odd] = g
    else:
        raise SystemExit(f"parity_report: no device generator for rows of kind {w.kind!r}")
    return x.to(tdt).contiguous()


def run(workload="cfg2", rows=100000, chunk=1024, threads=16, seed=20240607):
    """The comparison; returns the report as a dict."""
    args = argparse.Namespace(workload=workload, rows=rows, chunk=chunk, threads=threads, seed=seed)

    import torch

    import executorch_amd as ea
    from executorch_amd import workloads as W
    from oracle import oracle as O

    O.build()
    assert torch.cuda.is_available(), "parity_report.py needs a GPU"
    dev = torch.device("cuda:0")
    w = W.WORKLOADS[args.workload]
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed)
    inv = O.inv_temperature(w.temperature)
    s = ea.Sampler(w.vocab, w.temperature, w.topp, 1, max_batch=args.chunk)
    # the same rows through a call without debug records: pass 2 may then list only the largest
    # candidates of a peaked row, which must not change any token
    plain = ea.Sampler(w.vocab, w.temperature, w.topp, 1, max_batch=args.chunk)

    done = mismatches = plain_mismatches = sum_mismatches = tie_rows = tie_not_equal = native_agree = 0
    t0 = time.time()
    while done < args.rows:
        n = min(args.chunk, args.rows - done)
        x = device_rows(w, n, gen, torch, dev)
        seeds = (np.uint64(args.seed) + np.uint64(done) + np.arange(n, dtype=np.uint64) + np.uint64(1)).astype(np.uint64)
        s.set_rng_states(seeds)
        ddbg = torch.zeros((n, 8), dtype=torch.int32, device=dev)
        got = s.sample_batch(x, debug_out=ddbg).cpu().numpy()
        plain.set_rng_states(seeds)
        got_plain = plain.sample_batch(x).cpu().numpy()
        if w.dtype == W.DTYPE_BFLOAT16:
            host = np.ascontiguousarray(x.view(torch.int16).cpu().numpy().view(np.uint16))
        else:
            host = np.ascontiguousarray(x.cpu().numpy())
        want, ex = O.sample_rows(host, w.dtype, inv, w.topp, 0, seeds.copy(), mode=O.MODE_UPCAST, tie=O.TIE_STABLE,
                                 threads=args.threads, explain=True)
        sums = np.ascontiguousarray(ea.debug_records(ddbg)["sum"], dtype=np.float32)
        want_sums = np.array([ex[b].sum for b in range(n)], dtype=np.float32)
        sum_mismatches += int((sums.view(np.uint32) != want_sums.view(np.uint32)).sum())
        ref, ref_ex = O.sample_rows(host, w.dtype, inv, w.topp, 0, seeds.copy(), mode=O.MODE_UPCAST, tie=O.TIE_LIBSTDCXX,
                                    threads=args.threads, explain=True)
        native, _ = O.sample_rows(host, w.dtype, inv, w.topp, 0, seeds.copy(), mode=O.MODE_NATIVE, tie=O.TIE_LIBSTDCXX,
                                  threads=args.threads)
        mismatches += int((got != want).sum())
        plain_mismatches += int((got_plain != want).sum())
        native_agree += int((got == native).sum())
        for b in np.nonzero(ref != want)[0]:
            tie_rows += 1
            if ex[b].branch in (O.BRANCH_TOPP, O.BRANCH_TOPK):
                # both runs report the probability of the token they returned
                equal = np.float32(ex[b].p_token).view(np.uint32) == np.float32(ref_ex[b].p_token).view(np.uint32)
            else:
                po = np.empty(w.vocab, dtype=np.float32)
                o = O.Sampler(w.vocab, w.temperature, w.topp, 1, mode=O.MODE_UPCAST)
                o.sample(host[b].copy(), w.dtype, probs_out=po)
                equal = po[ref[b]] == po[want[b]]
            if not equal:
                tie_not_equal += 1
        done += n
        print(f"parity_report: {done} rows, {mismatches} + {plain_mismatches} mismatches, {time.time() - t0:.0f} s", file=sys.stderr,
              flush=True)

    return {
        "workload": f"{w.name}: vocab {w.vocab}, {W.DTYPE_NAMES[w.dtype]} ({w.kind}), temperature {w.temperature}, top-p {w.topp}",
        "rows": done,
        "token_mismatches_vs_oracle_fp32_index_ties": mismatches,
        "token_mismatches_without_debug_records": plain_mismatches,
        "normaliser_bit_mismatches_vs_oracle": sum_mismatches,
        "rows_differing_from_reference_tie_order": tie_rows,
        "of_which_not_between_equal_probabilities": tie_not_equal,
        "rows_equal_to_native_16bit_reference_arithmetic": native_agree,
        "seconds": round(time.time() - t0, 1),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="cfg2")
    ap.add_argument("--rows", type=int, default=100000)
    ap.add_argument("--chunk", type=int, default=1024)
    ap.add_argument("--threads", type=int, default=16)
    ap.add_argument("--seed", type=int, default=20240607)
    args = ap.parse_args()
    res = run(args.workload, args.rows, args.chunk, args.threads, args.seed)
    print(json.dumps(res))
    ok = res["token_mismatches_vs_oracle_fp32_index_ties"] == 0 and res["token_mismatches_without_debug_records"] == 0 and \
        res["normaliser_bit_mismatches_vs_oracle"] == 0 and \
        res["of_which_not_between_equal_probabilities"] == 0
    sys.exit(0 if ok else 1)


if __name__ == "__main__":
    main()
