#!/usr/bin/env python3
"""Index-math and quantizer kernels of the lookup path, timed one by one on one MI355X.

    python bench_index_ops.py [--config c2|c3|c5] [--steps K] [--warmup W] [--idx int32|int64]

For every operator of ``torchrec_amd.ops`` that sits around the lookup (offsets
scan, per-key totals, feature permutation, block bucketization, positions in
bags, position weights, row quantization) the script launches it K times through
the C ABI on synthetic inputs of the named workload's shape, brackets the
launches with HIP events on the launching stream and prints one JSON line:
algorithmic bytes per call (every input read once, every output written once),
microseconds per call, GB/s, and that rate as a fraction of what the plain copy
kernel (``tra_copy_bytes``, 256 MiB, timed in the same run) reaches.  A call
that consists of several launches (permute, bucketize) is timed as a whole; the
per-kernel durations are in the rocprofv3 summaries under ``profiles/``.

Shapes (the benchmark configurations): c2 = 26 features x B 2048, lengths U[1,40] with
5 % empty; c3 = 64 x 4096, Poisson(30); c5 = 8 x 16384, fixed 80.
"""
from __future__ import annotations

import argparse
import json
import sys

import numpy as np
import torch

from torchrec_amd import _lib


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--config", default="c3", choices=["c2", "c3", "c5"])
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--idx", default="int64", choices=["int32", "int64"], help="type of ids, lengths and offsets")
    p.add_argument("--buckets", type=int, default=8, help="world size of the bucketizer")
    p.add_argument("--quant-rows", type=int, default=1 << 20, help="rows of the quantizer input (x 128 fp32)")
    return p.parse_args()


def make_lengths(cfg: str, gen: np.random.Generator):
    if cfg == "c2":
        F, B = 26, 2048
        ln = gen.integers(1, 41, size=F * B)
        ln[gen.random(F * B) < 0.05] = 0
    elif cfg == "c3":
        F, B = 64, 4096
        ln = gen.poisson(30.0, size=F * B)
    else:
        F, B = 8, 16384
        ln = np.full(F * B, 80)
    return F, B, ln.astype(np.int64)


def main():
    args = parse_args()
    if not torch.cuda.is_available():
        sys.exit("bench_index_ops.py needs an MI355X GPU")
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    l = _lib.lib()
    gen = np.random.default_rng(7)
    F, B, ln = make_lengths(args.config, gen)
    n = F * B
    L = int(ln.sum())
    tdt = torch.int32 if args.idx == "int32" else torch.int64
    es = 4 if args.idx == "int32" else 8
    is64 = int(es == 8)
    rows_per_feature = 1_000_000
    lengths = torch.from_numpy(ln).to(dev, tdt)
    ids = torch.from_numpy(gen.integers(0, rows_per_feature, size=L)).to(dev, tdt)
    weights = torch.rand(L, device=dev, dtype=torch.float32)
    offsets = torch.zeros(n + 1, dtype=tdt, device=dev)
    offsets[1:] = torch.cumsum(lengths, 0)
    stream = _lib.current_stream(dev)
    P = _lib.ptr

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e3 / args.steps  # us

    # the copy kernel: the rate a plain stream reaches on this GPU
    nbytes = 256 << 20
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    copy_us = timed(lambda: _lib.check(l.tra_copy_bytes(P(src), P(dst), nbytes, stream)))
    copy_gbps = 2 * nbytes / copy_us / 1e3
    del src, dst
    results = []

    def report(name, us, nbytes_alg, launches, note=""):
        gbps = nbytes_alg / us / 1e3
        r = {
            "op": name, "config": args.config, "idx": args.idx, "us_per_call": round(us, 2),
            "algorithmic_bytes": int(nbytes_alg), "GBps": round(gbps, 1),
            "frac_of_copy_kernel": round(gbps / copy_gbps, 3), "launches": launches,
        }
        if note:
            r["note"] = note
        results.append(r)
        print(json.dumps(r), flush=True)

    # ---- offsets scan ------------------------------------------------------------------
    out_off = torch.empty(n + 1, dtype=tdt, device=dev)
    ws_bytes = l.tra_cumsum_workspace_bytes(n)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    us = timed(lambda: _lib.check(l.tra_cumsum(P(lengths), n, is64, P(out_off), P(ws), stream)))
    assert torch.equal(out_off, offsets)
    report("tra_cumsum", us, n * es + (n + 1) * es, "scan")

    # ---- per-key totals ----------------------------------------------------------------
    lpk = torch.empty(F, dtype=torch.int64, device=dev)
    us = timed(lambda: _lib.check(l.tra_length_per_key(P(lengths), F, B, is64, P(lpk), stream)))
    assert torch.equal(lpk, lengths.view(F, B).sum(1))
    report("tra_length_per_key", us, n * es + F * 8, "1")

    # ---- feature permutation (keys reversed) ----------------------------------------------
    perm = torch.arange(F - 1, -1, -1, dtype=torch.int32, device=dev)
    p_len = torch.empty(n, dtype=tdt, device=dev)
    us_l = timed(lambda: _lib.check(l.tra_permute_2d_lengths(P(perm), F, F, B, P(lengths), is64, P(p_len), stream)))
    assert torch.equal(p_len.view(F, B), lengths.view(F, B).flip(0))
    report("tra_permute_2d_lengths", us_l, 2 * n * es, "1")
    p_off = torch.zeros(n + 1, dtype=tdt, device=dev)
    p_off[1:] = torch.cumsum(p_len, 0)
    p_val = torch.empty(L, dtype=tdt, device=dev)
    p_w = torch.empty(L, dtype=torch.float32, device=dev)
    us_d = timed(lambda: _lib.check(l.tra_permute_2d_data(
        P(perm), F, B, P(offsets), P(p_off), is64, P(ids), es, P(weights), P(p_val), P(p_w), stream)))
    report("tra_permute_2d_data", us_d, 2 * L * (es + 4) + 2 * F * es, "1", "ids and weights")

    # ---- block bucketization --------------------------------------------------------------
    W = args.buckets
    bs = torch.full((F,), (rows_per_feature + W - 1) // W, dtype=torch.int64, device=dev)
    new_len = torch.empty(W * n, dtype=tdt, device=dev)
    us_bl = timed(lambda: _lib.check(l.tra_bucketize_lengths(
        P(offsets), P(ids), is64, P(bs), F, B, W, P(new_len), stream)))
    report("tra_bucketize_lengths", us_bl, (n + 1) * es + L * es + W * n * es, "1", f"{W} buckets")
    new_off = torch.zeros(W * n + 1, dtype=tdt, device=dev)
    new_off[1:] = torch.cumsum(new_len, 0)
    assert int(new_off[-1]) == L
    ws_bytes = l.tra_bucketize_workspace_bytes(F, B, W)
    cursor = torch.empty(ws_bytes // 8, dtype=torch.int64, device=dev) if ws_bytes else None
    new_ids = torch.empty(L, dtype=tdt, device=dev)
    new_w = torch.empty(L, dtype=torch.float32, device=dev)
    unb = torch.empty(L, dtype=torch.int64, device=dev)
    us_bs = timed(lambda: _lib.check(l.tra_bucketize_scatter(
        P(offsets), P(ids), is64, P(weights), P(bs), F, B, W, 0, P(new_off), P(cursor), P(new_ids), P(new_w),
        P(unb), stream)))
    report("tra_bucketize_scatter", us_bs,
           (n + 1) * es + W * n * es + L * (es + 4) + L * (es + 4) + L * 8, "1",
           f"{W} buckets, weights and unbucketize_permute")

    # ---- positions in bags, position weights --------------------------------------------------
    rng_out = torch.empty(L, dtype=tdt, device=dev)
    us = timed(lambda: _lib.check(l.tra_offsets_range(P(offsets), n, is64, L, P(rng_out), stream)))
    report("tra_offsets_range", us, n * es + L * es, "1")
    max_len = int(ln.max()) + 1
    key_start = torch.arange(F, dtype=torch.int32, device=dev) * max_len
    key_len = torch.full((F,), max_len, dtype=torch.int32, device=dev)
    table = torch.rand(F * max_len, dtype=torch.float32, device=dev)
    pw = torch.empty(L, dtype=torch.float32, device=dev)
    us = timed(lambda: _lib.check(l.tra_position_weights(
        P(offsets), is64, F, B, P(key_start), P(key_len), P(table), P(pw), stream)))
    report("tra_position_weights", us, (n + 1) * es + L * 4, "1")

    # ---- row quantizer ---------------------------------------------------------------------------
    R, D = args.quant_rows, 128
    x = torch.randn(R, D, device=dev, dtype=torch.float32)
    for bits in (8, 4, 2):
        rb = (D * bits // 8 + 4 + 15) // 16 * 16
        q = torch.empty(R, rb, dtype=torch.uint8, device=dev)
        us = timed(lambda: _lib.check(l.tra_quantize_rows(P(x), R, D, bits, P(q), rb, stream)))
        report(f"tra_quantize_rows int{bits}", us, R * D * 4 + R * (D * bits // 8 + 4), "1", f"{R} rows x {D}")

    print(json.dumps({"copy_kernel_GBps": round(copy_gbps, 1), "copy_us": round(copy_us, 2),
                      "shape": {"features": F, "batch": B, "bags": n, "ids": L}, "ops": len(results)}))


if __name__ == "__main__":
    main()
