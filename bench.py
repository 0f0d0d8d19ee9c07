#!/usr/bin/env python3
"""Benchmark of the quantized embedding inference path on one MI355X.

Default workload ("c2", the configuration the headline metric is quoted on):
DLRM-style pooled inference, 26 features / 26 tables, rows log-uniform in
[1e3, 4e7], dim 128, int4 row-wise with fp16 scale/bias, SUM pooling, fp16
output, batch 2048, bag lengths U[1, 40] with 5 % forced empty, ids
Zipf(1.05) over a seeded permutation of each table's rows.  Synthetic, seeded.

A step is one QuantEmbeddingBagCollection.forward over one KeyedJaggedTensor
(lengths -> offsets scan + the pooled lookup), inputs resident in HBM; steps
rotate over --batches distinct id batches.  The timed loop makes the plain
Python calls (--mode graph captures each batch's forward in a HIP graph and
replays the graphs instead; on this stack a graph launch costs more than the
two kernel launches it replaces, so it is not the default).

One JSON line is printed: the metric (pooled lookups/s), the roofline of the
lookup kernel (algorithmic bytes / HIP-event duration against 8 TB/s) and the
CPU baseline (fbgemm's own kernels on the host cores, bounded sample).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
CAL_COPY_BYTES = 1 << 28


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=2000)
    p.add_argument("--warmup", type=int, default=200)
    p.add_argument("--config", default="c2", choices=["c1", "c2", "c3", "c4", "c5"])
    p.add_argument("--batches", type=int, default=None,
                   help="distinct id batches rotated through (default 32 for c2, 12 for c4, 8 elsewhere)")
    p.add_argument("--mode", default="eager", choices=["graph", "eager"])
    p.add_argument("--split-bags", type=int, default=1,
                   help="c5 only: cut every bag of 80 into N bags of 80/N (bounds what splitting long bags could gain)")
    p.add_argument("--row-alignment", type=int, default=None, help="default 16 (TorchRec's), 4 for c5 (68-byte rows)")
    p.add_argument("--row-padding", default=None, choices=["line", "none"],
                   help="distance between rows in the packed store: 'line' = rows of at most 128 bytes at the next "
                        "power-of-two stride, so that none straddles a 128-byte line (the operator's default while the "
                        "padded store fits its budget); 'none' = at their width, the reference's layout")
    p.add_argument("--no-alt-layout", action="store_true",
                   help="c2 also measures the same workload with the other row padding; this skips it")
    p.add_argument("--request-streams", type=int, default=3,
                   help="also time the same steps dealt round-robin to this many HIP streams (independent "
                        "requests in flight); 0 or 1 = skip")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-pcie", action="store_true",
                   help="skip the leg that feeds every step from pinned host memory (profiling runs: the kernel "
                        "averages then cover launches with resident inputs only)")
    p.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU baseline sample")
    p.add_argument("--rocprof-summary", metavar="DIR", default=None,
                   help="no benchmark: summarize rocprofv3 CSV output under DIR (kernel_stats / counter_collection) "
                        "for this library's kernels and exit")
    p.add_argument("--id-permutation", default="fixed", choices=["fixed", "per-batch"],
                   help="c2: rank -> id through one seeded permutation per table shared by all batches (the named "
                        "workload), or through a new permutation for every batch (cold head: no row is hot in two "
                        "batches; a lower bound, not the named workload)")
    p.add_argument("--traffic-json", action="store_true",
                   help="with --rocprof-summary DIR: also write profiles/<config>_lookup_traffic.json from the "
                        "FETCH_SIZE / WRITE_SIZE runs under DIR, stamped with the hash of the kernel sources")
    p.add_argument("--batch-size", type=int, default=None, help="override the workload's batch size (tuning only; result is then not the named workload)")
    p.add_argument("--scale", type=float, default=1.0, help="shrink table rows (debug only; result is then invalid)")
    return p.parse_args()


# --------------------------------------------------------------------------
# workloads
# --------------------------------------------------------------------------
class ZipfTable:
    """Id source of one table: rank ~ truncated Zipf(alpha) on [1, rows], id = perm[rank - 1].

    The permutation is drawn ONCE per table, from a generator seeded by (workload
    seed, table), and every batch draws its ids through it: the hot rows of a
    table are the same rows in every batch, as they are for a model in service.
    Only the ranks differ from batch to batch."""

    def __init__(self, rows, alpha, seed, table, device):
        import torch

        g = torch.Generator(device=device)
        g.manual_seed(seed * 1_000_003 + table)
        self.rows = rows
        w = torch.arange(1, rows + 1, dtype=torch.float64, device=device).pow_(-alpha)
        cdf = torch.cumsum(w, 0)
        cdf /= cdf[-1].clone()
        self.cdf = cdf
        self.perm = torch.randperm(rows, device=device, generator=g).to(torch.int32)

    def draw(self, n, gen, fresh_permutation=False):
        import torch

        if fresh_permutation:  # the rows that are hot change with every batch (no reuse from batch to batch)
            self.perm = torch.randperm(self.rows, device=self.perm.device, generator=gen).to(torch.int32)
        if n == 0:
            return torch.zeros(0, dtype=torch.int64, device=self.perm.device)
        u = torch.rand(n, dtype=torch.float64, device=self.perm.device, generator=gen)
        rank = torch.searchsorted(self.cdf, u).clamp_(max=self.rows - 1)
        return self.perm[rank].long()

    def hottest(self, k):
        """The ids of ranks 1..k."""
        return self.perm[:k].long()


def build_workload(args, dev):
    """Returns dict(module, batches=[(values, lengths, weights)], keys, meta...)."""
    import numpy as np
    import torch

    from torchrec_amd import _lib
    from torchrec_amd.modules.embedding_configs import DataType, EmbeddingBagConfig, EmbeddingConfig, PoolingType
    from torchrec_amd.quant import EmbeddingBagCollection as QuantEBC, EmbeddingCollection as QuantEC

    cfg = args.config
    seed = 1000 + int(cfg[1])
    rng = np.random.default_rng(seed)
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    DT = {"int8": DataType.INT8, "int4": DataType.INT4, "int2": DataType.INT2, "fp16": DataType.FP16}

    weighted, pooled, out_dtype, pooling = False, True, torch.half, PoolingType.SUM
    zipf = None
    if cfg == "c1":
        T, B = 8, 512
        rows = [100_000] * T
        dims, dts = [64] * T, ["int8"] * T
        lens = lambda: np.full(T * B, 20, dtype=np.int64)
        id_fn = lambda n, r, t: torch.randint(0, r, (n,), device=dev, generator=gen)
        desc = "c1: QEBC 8 tables x 100k x 64 int8, B512, L=20, SUM, fp16 out, uniform ids"
    elif cfg == "c2":
        T, B = 26, 2048
        rows = [max(1000, int(round(math.exp(x) * args.scale))) for x in rng.uniform(math.log(1e3), math.log(4e7), T)]
        dims, dts = [128] * T, ["int4"] * T

        def lens():
            l = rng.integers(1, 41, T * B)
            l[rng.random(T * B) < 0.05] = 0
            return l

        zipf = [ZipfTable(rows[t], 1.05, seed, t, dev) for t in range(T)]
        fresh = getattr(args, "id_permutation", "fixed") == "per-batch"
        id_fn = lambda n, r, t: zipf[t].draw(n, gen, fresh)
        desc = ("c2: QEBC 26 tables rows logU[1e3,4e7] x 128 int4, B2048, len U[1,40] 5% empty, Zipf(1.05) over one "
                "seeded permutation per table (the same in every batch), SUM, fp16 out")
    elif cfg == "c3":
        T, B = 64, 4096
        rows = [max(1000, int(round(math.exp(x) * args.scale))) for x in rng.uniform(math.log(1e5), math.log(1e7), T)]
        dims = [[32, 64, 128, 256][t % 4] for t in range(T)]
        dts = [["int8", "int4", "int2", "fp16"][(t // 4) % 4] for t in range(T)]
        lens = lambda: rng.poisson(30, T * B)
        id_fn = lambda n, r, t: torch.randint(0, r, (n,), device=dev, generator=gen)
        weighted, out_dtype = True, torch.float
        desc = "c3: QEBC 64 tables mixed D{32..256} x {int8,int4,int2,fp16}, B4096, Poisson(30), weighted SUM, fp32 out"
    elif cfg == "c4":
        T, B = 16, 1024
        rows = [max(1000, int(1_000_000 * args.scale))] * T
        dims, dts = [128] * T, ["int8"] * T
        lens = lambda: rng.integers(0, 257, T * B)
        id_fn = lambda n, r, t: torch.randint(0, r, (n,), device=dev, generator=gen)
        pooled = False
        desc = "c4: QEC 16 tables x 1e6 x 128 int8, B1024, len U[0,256], uniform ids, jagged fp16 out"
    else:
        T, B = 8, 16384
        rows = [max(1000, int(250_000_000 * args.scale))] * T
        dims, dts = [128] * T, ["int4"] * T
        # --split-bags N: every bag of 80 cut into N bags of 80 / N (N x the bags, the same ids in the same
        # order): what a lookup that splits long bags over N lane groups would pool before its
        # cross-lane reduction, i.e. a lower bound on that variant's time.
        split = max(1, int(getattr(args, "split_bags", 1) or 1))
        if 80 % split:
            raise SystemExit("--split-bags must divide 80")
        B *= split
        lens = lambda: np.full(T * B, 80 // split, dtype=np.int64)
        pooling = PoolingType.MEAN
        id_fn = None  # affine bijection below: a 250M-entry permutation per table is not needed
        desc = "c5: QEBC 8 tables x 250M x 128 int4 (68 B rows), B16384, L=80, Zipf(0.8), MEAN, fp16 out"
        if split > 1:
            desc += f" [every bag split into {split} bags of {80 // split}: B{B}; not the c5 workload]"

    if getattr(args, "batch_size", None):
        B = args.batch_size
        desc += f" [batch size overridden to {B}]"
    from torchrec_amd import tbe as _tbe
    # (c5 is by definition the 68-byte stride: its shortened test shapes must not be padded either)
    previous_padding = _tbe.set_default_row_padding(
        getattr(args, "row_padding", None) or ("none" if cfg == "c5" else _tbe.get_default_row_padding()))
    if pooled:
        tables = [
            EmbeddingBagConfig(name=f"t{t}", embedding_dim=dims[t], num_embeddings=rows[t], feature_names=[f"f{t}"],
                               data_type=DT[dts[t]], pooling=pooling)
            for t in range(T)
        ]
        module = QuantEBC(tables, weighted, dev, output_dtype=out_dtype, row_alignment=args.row_alignment)
    else:
        tables = [
            EmbeddingConfig(name=f"t{t}", embedding_dim=dims[t], num_embeddings=rows[t], feature_names=[f"f{t}"],
                            data_type=DT[dts[t]])
            for t in range(T)
        ]
        module = QuantEC(tables, dev, output_dtype=out_dtype, row_alignment=args.row_alignment)
    _tbe.set_default_row_padding(previous_padding)

    # Fill the packed store: fp32 N(0, 0.1) rows quantized on the GPU, chunk by chunk,
    # straight into their header-first rows (c5: synthetic packed bytes, no float master).
    lib = _lib.lib()
    stream = _lib.current_stream(dev)
    BITS = {"int8": 8, "int4": 4, "int2": 2}
    for tbe in module._emb_modules:
        for t, name in enumerate(tbe.embedding_names):
            gt = int(name[1:])
            view = tbe._rows_view(t)
            r, rb = tbe.rows[t], tbe.row_stride[t]  # distance between rows in the packed store
            step = max(1, (1 << 27) // dims[gt])
            for r0 in range(0, r, step):
                n = min(step, r - r0)
                if cfg == "c5":
                    chunk = view[r0:r0 + n]
                    chunk[:, 4:4 + dims[gt] // 2] = torch.randint(0, 256, (n, dims[gt] // 2), dtype=torch.uint8, device=dev, generator=gen)
                    sc = torch.empty(n, device=dev).uniform_(0.004, 0.02, generator=gen).half()
                    bi = torch.empty(n, device=dev).uniform_(-0.15, -0.03, generator=gen).half()
                    chunk[:, 0:2] = sc.view(torch.uint8).view(n, 2)
                    chunk[:, 2:4] = bi.view(torch.uint8).view(n, 2)
                    continue
                w = torch.empty((n, dims[gt]), device=dev).normal_(0, 0.1, generator=gen)
                if dts[gt] == "fp16":
                    view[r0:r0 + n, : 2 * dims[gt]] = w.half().view(torch.uint8)
                else:
                    dst = tbe.weights_dev.data_ptr() + tbe.weights_physical_offsets[t] + r0 * rb
                    _lib.check(lib.tra_quantize_rows(_lib.ptr(w), n, dims[gt], BITS[dts[gt]], dst, rb, stream))
                torch.cuda.synchronize(dev)
                del w

    batches = []
    for _ in range(args.batches):
        l = lens().astype(np.int64)
        per = l.reshape(T, B).sum(axis=1)
        if cfg == "c5":
            vals = []
            for t in range(T):
                n, N = int(per[t]), rows[t]
                # rank ~ truncated Zipf(0.8) by inverse CDF of the continuous envelope, then an affine bijection
                u = torch.rand(n, dtype=torch.float64, device=dev, generator=gen)
                a = 1.0 - 0.8
                rank = ((u * ((N + 1.0) ** a - 1.0) + 1.0).pow_(1.0 / a) - 1.0).long().clamp_(0, N - 1)
                mul = 2654435761 % N
                while math.gcd(mul, N) != 1:
                    mul += 1
                vals.append((rank * mul + 12345 * (t + 1)) % N)
            values = torch.cat(vals)
        else:
            values = torch.cat([id_fn(int(per[t]), rows[t], t) for t in range(T)])
        values = values.to(torch.int32)
        lengths = torch.from_numpy(l).to(torch.int32).to(dev)
        w = torch.rand(values.numel(), device=dev, generator=gen) if weighted else None
        batches.append((values, lengths, w))
    torch.cuda.synchronize(dev)
    hot_ids = None
    if zipf is not None:
        hot_ids = [z.hottest(min(16, z.rows)) for z in zipf]
        if fresh:
            desc = desc.replace("one seeded permutation per table (the same in every batch)",
                                "a NEW permutation per table for every batch (cold head)")
        del zipf, id_fn

    # algorithmic bytes per call: unpadded rows + ids + weights + offsets + output
    def alg_bytes(values, lengths):
        per = lengths.view(T, B).sum(dim=1).tolist()
        row_b = 0
        for t in range(T):
            bits = {"int8": 8, "int4": 4, "int2": 2, "fp16": 16}[dts[t]]
            row_b += per[t] * (dims[t] * bits // 8 + (4 if dts[t] != "fp16" else 0))
        L = values.numel()
        osz = 2 if out_dtype == torch.half else 4
        out_b = (B * sum(dims) if pooled else L * dims[0]) * osz
        return row_b + 4 * L + (4 * L if weighted else 0) + 4 * (T * B + 1) + out_b

    return dict(
        module=module, batches=batches, keys=[f"f{t}" for t in range(T)], T=T, B=B, rows=rows, dims=dims, dts=dts,
        weighted=weighted, pooled=pooled, out_dtype=out_dtype, desc=desc, hot_ids=hot_ids,
        alg_bytes=[alg_bytes(v, l) for v, l, _ in batches],
        store_bytes=sum(m.weights_size for m in module._emb_modules),
    )


# --------------------------------------------------------------------------
# CPU baseline (fbgemm kernels from libtorch_cpu on the host cores)
# --------------------------------------------------------------------------
def cpu_baseline(wl, out_gpu, seconds):
    """fbgemm's CPU kernels (the ones the reference's CPU path runs) over the same
    batches, bags split over the host threads.  The whole packed store is copied
    to host memory when it fits; otherwise only the rows the batches touch."""
    import numpy as np
    import torch

    import oracle as O

    module = wl["module"]
    tbe = module._emb_modules[0]
    code = {"fp32": O.FP32, "fp16": O.FP16, "int8": O.INT8, "int4": O.INT4, "int2": O.INT2}
    T, B = wl["T"], wl["B"]
    NB = len(wl["batches"])
    host = []
    for values, lengths, w in wl["batches"]:
        offs = np.zeros(T * B + 1, dtype=np.int32)
        offs[1:] = np.cumsum(lengths.cpu().numpy())
        host.append([values.cpu().numpy(), offs, None if w is None else w.cpu().numpy()])
    try:
        avail = os.sysconf("SC_AVPHYS_PAGES") * os.sysconf("SC_PAGE_SIZE")
    except (ValueError, OSError):
        avail = 0
    whole = tbe.weights_size * 1.3 < avail and tbe.weights_size < 64e9
    if whole:
        store = O.Store(
            tbe.weights_dev.cpu().numpy(),
            np.asarray(tbe.weights_physical_offsets, dtype=np.int64), np.asarray(tbe.rows, dtype=np.int64),
            np.asarray(tbe.dims, dtype=np.int32), np.asarray([code[str(x)] for x in tbe.weight_tys], dtype=np.int32),
            np.asarray(tbe.row_stride, dtype=np.int32),
        )
        where = f"whole {tbe.weights_size / 1e9:.2f} GB store in host memory"
    else:
        # compact the rows any batch touches (the store does not fit the host)
        pieces, offsets_t, rows_t, base = [], [], [], 0
        for t in range(T):
            segs = [h[0][h[1][t * B]: h[1][(t + 1) * B]] for h in host]
            uniq = np.unique(np.concatenate(segs))
            for h in host:
                lo, hi = h[1][t * B], h[1][(t + 1) * B]
                h[0][lo:hi] = np.searchsorted(uniq, h[0][lo:hi])
            rb = tbe.row_bytes[t]
            view = tbe._rows_view(t)
            rows = view[torch.from_numpy(uniq.astype(np.int64)).to(view.device)].cpu().numpy() if len(uniq) else np.zeros((0, rb), np.uint8)
            pieces.append(rows.reshape(-1))
            offsets_t.append(base)
            rows_t.append(len(uniq))
            base += O.round_up(rows.size, 128)
            pieces.append(np.zeros(base - offsets_t[-1] - rows.size, dtype=np.uint8))
        store = O.Store(
            np.concatenate(pieces), np.asarray(offsets_t, dtype=np.int64), np.asarray(rows_t, dtype=np.int64),
            np.asarray(tbe.dims, dtype=np.int32), np.asarray([code[str(x)] for x in tbe.weight_tys], dtype=np.int32),
            np.asarray(tbe.row_bytes, dtype=np.int32),
        )
        where = (f"store too large for the host: tables compacted to the {int(sum(rows_t))} rows the batches touch "
                 f"({base / 1e9:.2f} GB), which flatters the CPU's cache hit rate")
    pooling = int(tbe.pooling_mode)
    odt = O.FP16 if wl["out_dtype"] == torch.half else O.FP32
    nthreads = max(1, min(16, len(os.sched_getaffinity(0))))
    ftm = list(tbe.feature_table_map)
    call = lambda i: O.tbe_forward(store, ftm, B, host[i][0], host[i][1], host[i][2], pooling, odt, "fbgemm", nthreads)
    ref = call(0)  # warm-up (fbgemm generates its kernels on first use) and the output that is compared
    t0, reps, done = time.perf_counter(), 0, 0
    while True:
        call(reps % NB)
        done += host[reps % NB][0].size
        reps += 1
        el = time.perf_counter() - t0
        if el > seconds:
            break
    got = out_gpu.cpu().numpy()
    if not wl["pooled"]:
        ref = ref[: got.shape[0]]  # rows of the first feature
    view = np.uint16 if got.dtype == np.float16 else np.uint32
    mism = int((got.view(view) != ref.view(view)).sum())
    return {
        "value": done / el,
        "unit": "lookups/s",
        "cores": nthreads,
        "kind": "reference",
        "sample": f"{reps} forwards over the same {NB} batches ({done} lookups) in {el:.1f} s; fbgemm "
                  f"GenerateEmbeddingSpMDM[NBit]WithStrides from libtorch_cpu (the kernels behind the reference's CPU "
                  f"TBE), bags split over {nthreads} threads; {where}",
        "gpu_vs_cpu_mismatching_outputs": mism,
        "outputs_compared": int(got.size),
    }


# --------------------------------------------------------------------------
# rocprofv3 output -> short text (the summaries kept under profiles/)
# --------------------------------------------------------------------------
def kernel_source_hash():
    """Hash of the sources the kernel library is built from (``torchrec_amd/csrc`` and
    ``include``): a stored hardware-counter profile names the hash it was measured at, and a
    bench run says whether the tree still has it."""
    import glob
    import hashlib

    h = hashlib.sha256()
    files = sorted(
        f for pat in ("torchrec_amd/csrc/*.hip", "torchrec_amd/csrc/*.h", "torchrec_amd/csrc/Makefile", "include/*.h")
        for f in glob.glob(os.path.join(ROOT, pat))
    )
    for f in files:
        h.update(os.path.relpath(f, ROOT).encode())
        h.update(b"\0")
        h.update(open(f, "rb").read())
        h.update(b"\0")
    return h.hexdigest()[:16]


def write_traffic_json(root, config):
    """``profiles/<config>_lookup_traffic.json`` from the FETCH_SIZE / WRITE_SIZE counter runs under
    ``root`` (as ``--rocprof-summary`` reads them): HBM bytes per lookup call = the counters of the
    lookup kernel instances of the timed step (those dispatched most often; a call launches each
    once), scaled by what the same counters read for the library's 256 MiB copy kernel."""
    import collections
    import csv
    import glob

    per = collections.defaultdict(lambda: collections.defaultdict(list))
    for f in sorted(glob.glob(os.path.join(root, "**", "*counter_collection.csv"), recursive=True)):
        for r in csv.DictReader(open(f)):
            if r["Counter_Name"] in ("FETCH_SIZE", "WRITE_SIZE"):
                per[r["Counter_Name"]][r["Kernel_Name"].split("(")[0].replace("void ", "")].append(float(r["Counter_Value"]))
    out = {}
    for ctr, copied_kib in (("FETCH_SIZE", CAL_COPY_BYTES / 1024), ("WRITE_SIZE", CAL_COPY_BYTES / 1024)):
        ks = per.get(ctr)
        if not ks:
            raise SystemExit(f"no {ctr} counters under {root}")
        copy = [v for k, v in ks.items() if "tra_copy_kernel" in k]
        if not copy:
            raise SystemExit(f"the {ctr} run has no dispatch of the calibration copy kernel")
        factor = copied_kib / (sum(copy[0]) / len(copy[0]))
        lookups = {k: v for k, v in ks.items() if "tbe_pooled" in k or "tbe_nobag" in k}
        most = max(len(v) for v in lookups.values())
        step = {k: sum(v) / len(v) for k, v in lookups.items() if len(v) == most}
        out[ctr] = (sum(step.values()) * 1024 * factor, factor, sorted(step))
    fetch, ff, kernels = out["FETCH_SIZE"]
    write, wf, _ = out["WRITE_SIZE"]
    doc = {
        "kernel": kernels if len(kernels) > 1 else kernels[0],
        "workload": config,
        "hbm_bytes_per_launch": int(round(fetch + write)),
        "fetch_bytes": int(round(fetch)),
        "write_bytes": int(round(write)),
        "fetch_factor": round(ff, 4),
        "write_factor": round(wf, 4),
        "kernel_source_hash": kernel_source_hash(),
        "note": "per lookup call (all its launches); counter x factor, the factor from the same counter over the "
                "256 MiB copy kernel; kernel_source_hash covers torchrec_amd/csrc and include",
    }
    path = os.path.join(ROOT, "profiles", f"{config}_lookup_traffic.json")
    with open(path, "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")
    print(f"wrote {os.path.relpath(path, ROOT)}: {doc['hbm_bytes_per_launch'] / 1e6:.1f} MB per call")


def rocprof_summary(root):
    import collections
    import csv
    import glob

    mine = lambda name: "tbe_" in name or "tra_" in name or "tra::" in name
    short = lambda name: name.split("(")[0].replace("void ", "")[:100]
    for f in sorted(glob.glob(os.path.join(root, "**", "*kernel_stats.csv"), recursive=True)):
        print(f"# {os.path.relpath(f, root)}")
        print(f"{'calls':>8s} {'avg_us':>10s} {'min_us':>10s} {'max_us':>10s} {'pct':>7s}  kernel")
        for r in csv.DictReader(open(f)):
            if mine(r["Name"]):
                print(f"{int(r['Calls']):8d} {float(r['AverageNs']) / 1e3:10.2f} {float(r['MinNs']) / 1e3:10.2f} "
                      f"{float(r['MaxNs']) / 1e3:10.2f} {float(r['Percentage']):7.2f}  {short(r['Name'])}")
    for f in sorted(glob.glob(os.path.join(root, "**", "*counter_collection.csv"), recursive=True)):
        agg = collections.defaultdict(list)
        for r in csv.DictReader(open(f)):
            if mine(r["Kernel_Name"]):
                agg[(short(r["Kernel_Name"]), r["Counter_Name"])].append(float(r["Counter_Value"]))
        print(f"# {os.path.relpath(f, root)}")
        print(f"{'dispatches':>10s} {'mean per dispatch':>20s}  counter  kernel")
        for (k, c), v in sorted(agg.items()):
            print(f"{len(v):10d} {sum(v) / len(v):20.1f}  {c}  {k}")


KERNEL_MIN_LAUNCHES = 200
KERNEL_MIN_WARMUP = 500


def time_kernel_launches(fn, steps, warmup, nb):
    """Average period of a lookup launch in a queue that stays full: ``fn(batch)``
    is launched ``max(warmup, 500)`` times untimed, then, with no wait in between,
    ``max(steps, 200)`` times between two HIP events recorded on the launching
    stream.  The first event is reached when the last untimed launch ends, the
    second when the last timed one ends, so the quotient is the steady-state time
    per launch (its kernel plus the gap to the next one).  The counts have floors
    because the quantity is a property of the kernel, not of the run's length: a
    region of 20 launches that opens on a GPU which has idled through set-up reads
    1 to 2 us more per 24 us launch than the same launches deep inside a long run
    (the first few hundred launches after an idle stretch are slower), and that
    start-up belongs to ``ms_per_step``, whose region does open so.
    Returns (ms per launch, launches timed)."""
    import torch

    n = max(steps, KERNEL_MIN_LAUNCHES)
    torch.cuda.synchronize()
    for k in range(max(warmup, KERNEL_MIN_WARMUP)):
        fn(k % nb)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for k in range(n):
        fn(k % nb)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / n, n


def measure_alt_layout(args, dev, row_padding, ref_out):
    """The same workload (same seeds: same tables, same ids) stored with the other
    row padding: step time of the module forward, kernel time of its lookup
    launch, and whether the outputs equal those of the headline layout."""
    import argparse as _ap
    import torch
    from torchrec_amd import _lib, KeyedJaggedTensor

    alt = _ap.Namespace(**vars(args))
    alt.row_padding = row_padding
    wl = build_workload(alt, dev)
    module, batches, keys = wl["module"], wl["batches"], wl["keys"]
    NB = len(batches)

    def forward(i):
        v, l, w = batches[i]
        return module(KeyedJaggedTensor(keys=keys, values=v, lengths=l, weights=w))

    out0 = forward(0)
    torch.cuda.synchronize()
    same = bool(torch.equal(out0.values(), ref_out))
    steps, warm = args.steps, min(args.warmup, 200)
    for k in range(warm):
        forward(k % NB)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        forward(k % NB)
    torch.cuda.synchronize()
    el = time.perf_counter() - t0
    tbe = module._emb_modules[0]
    lib = _lib.lib()
    plan = tbe._get_plan(None)
    stream = _lib.current_stream(dev)
    kout = out0.values().clone()
    ws = torch.empty(max(256, lib.tra_tbe_forward_lengths_workspace_bytes(wl["T"], wl["B"], 0)), dtype=torch.uint8, device=dev)
    info = ctypes.create_string_buffer(4096)
    _lib.check(lib.tra_tbe_launch_info(plan, wl["B"], batches[0][0].numel(), int(tbe.pooling_mode), wl["T"], info, len(info)))
    launches = info.value.decode().split("; ")

    def launch(i):
        v, l, w = batches[i]
        _lib.check(lib.tra_tbe_forward_lengths(plan, _lib.ptr(tbe.weights_dev), _lib.ptr(v), _lib.ptr(l), 0, _lib.ptr(w),
                                               wl["B"], wl["T"], v.numel(), int(tbe.pooling_mode), tbe.output_dtype,
                                               _lib.ptr(kout), kout.stride(0), _lib.ptr(ws), stream))

    call_ms, timed_launches = time_kernel_launches(launch, steps, warm, NB)
    alg = sum(wl["alg_bytes"][k % NB] for k in range(timed_launches)) / timed_launches
    lookups = sum(batches[k % NB][0].numel() for k in range(steps))
    return {
        "row_padding": row_padding,
        "row_stride_bytes": sorted(set(wl["module"]._emb_modules[0].row_stride)),
        "store_GB": wl["store_bytes"] / 1e9,
        "value": lookups / el, "unit": "lookups/s", "ms_per_step": el / steps * 1e3,
        "lookup_call_ms": call_ms, "launches_timed": timed_launches, "launches_per_call": launches,
        "achieved": alg / (call_ms * 1e-3) / 1e9, "frac": alg / (call_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "outputs_equal_headline_layout": same,
        "note": "same tables and ids, rows stored with the other row padding ('none' = rows at their width, the "
                "reference's layout; 'line' = power-of-two stride, no row straddles a 128-byte line); algorithmic "
                "bytes unchanged (unpadded rows); lookup_call_ms covers the whole lookup call "
                "(tra_tbe_forward_lengths), scan kernels included when it is not fused",
    }


def main():
    args = parse_args()
    if args.rocprof_summary:
        rocprof_summary(args.rocprof_summary)
        if args.traffic_json:
            write_traffic_json(args.rocprof_summary, args.config)
        return
    if args.row_alignment is None:
        args.row_alignment = 4 if args.config == "c5" else 16
    if args.batches is None:
        # (c4: more distinct id counts than the plan keeps launch geometries, so that a geometry
        # that is looked up per exact id count would show as a miss on every call)
        args.batches = {"c2": 32, "c4": 12}.get(args.config, 8)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    from torchrec_amd import _lib, KeyedJaggedTensor

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    _lib.lib()  # fail early if the kernel library is missing

    t_setup = time.time()
    wl = build_workload(args, dev)
    module, batches, keys = wl["module"], wl["batches"], wl["keys"]
    NB = len(batches)
    print(f"[bench] {wl['desc']}; store {wl['store_bytes'] / 1e9:.2f} GB; setup {time.time() - t_setup:.1f} s",
          file=sys.stderr, flush=True)

    def forward(i):
        v, l, w = batches[i]
        return module(KeyedJaggedTensor(keys=keys, values=v, lengths=l, weights=w))

    def out_tensor(o):
        return o.values() if wl["pooled"] else next(iter(o.values())).values()

    # eager warm-up (creates the launch plans), then optional graph capture
    outs = [forward(i) for i in range(NB)]
    torch.cuda.synchronize()
    graphs = None
    if args.mode == "graph" and not wl["pooled"]:
        print("bench.py: --mode graph needs a forward without host reads; the sequence collection fetches its "
              "per-feature row counts on the host (as the reference does), use --mode eager", file=sys.stderr)
        sys.exit(2)
    if args.mode == "graph":
        graphs, gouts = [], []
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for i in range(NB):
                forward(i)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        for i in range(NB):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                o = forward(i)
            graphs.append(g)
            gouts.append(o)
        torch.cuda.synchronize()
        # replays must reproduce the eager result exactly
        for i in range(NB):
            graphs[i].replay()
        torch.cuda.synchronize()
        for i in range(NB):
            if not torch.equal(out_tensor(gouts[i]), out_tensor(outs[i])):
                raise RuntimeError(f"graph replay of batch {i} differs from the eager forward")

    def run(mode, steps):
        if mode == "graph":
            for k in range(steps):
                graphs[k % NB].replay()
        else:
            for k in range(steps):
                forward(k % NB)

    def timed(mode, steps, warmup):
        run(mode, warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(mode, steps)
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    tbe0 = module._emb_modules[0]
    lookups = [b[0].numel() for b in batches]
    total_lookups = sum(lookups[k % NB] for k in range(args.steps))
    el = timed(args.mode, args.steps, args.warmup)
    other = "eager" if args.mode == "graph" else None
    el_other = timed("eager", args.steps, min(args.warmup, 50)) if other else None
    # host-side cost of a step: the same loop without waiting for the GPU
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    host_steps = min(max(args.steps, 200), 500)
    run("eager", host_steps)
    host_ms = (time.perf_counter() - t0) / host_steps * 1e3
    torch.cuda.synchronize()

    # ---- the same step fed from pinned host memory (ids, lengths, weights cross PCIe every step)
    pinned = [tuple(None if t is None else t.cpu().pin_memory() for t in b) for b in batches]
    big = max(range(NB), key=lambda i: batches[i][0].numel())  # staging buffers hold the largest batch
    dev_in = [tuple(None if t is None else torch.empty_like(t) for t in batches[big]) for _ in range(2)]

    def forward_from_host(k):
        src, dst = pinned[k % NB], dev_in[k % 2]
        for s_, d_ in zip(src, dst):
            if s_ is not None:
                d_[: s_.numel()].copy_(s_, non_blocking=True)
        v, l, w = dst
        n = src[0].numel()
        return module(KeyedJaggedTensor(keys=keys, values=v[:n], lengths=l, weights=None if w is None else w[:n]))

    hsteps = 0 if args.no_pcie else min(args.steps, 500)
    el_host, host_lookups = 0.0, 0
    if hsteps:
        for k in range(20):
            forward_from_host(k)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(hsteps):
            forward_from_host(k)
        torch.cuda.synchronize()
        el_host = time.perf_counter() - t0
        host_lookups = sum(lookups[k % NB] for k in range(hsteps))

    # ---- kernel-only timing: the lookup launch(es) alone, HIP events on the launch stream
    tbe = module._emb_modules[0]
    lib = _lib.lib()
    offs = []
    from torchrec_amd import ops
    for v, l, w in batches:
        offs.append(ops.asynchronous_complete_cumsum(l))
    if wl["pooled"]:
        kout = out_tensor(outs[0]).clone()
    else:
        # sequence lookup writes one row per id of every feature: [max L, D]
        odt = torch.half if wl["out_dtype"] == torch.half else torch.float
        kout = torch.empty(max(b[0].numel() for b in batches), wl["dims"][0], dtype=odt, device=dev)
    if len(module._emb_modules) != 1:
        raise RuntimeError("bench.py times one lookup operator; this workload built several")
    stream = _lib.current_stream(dev)
    plan = tbe._get_plan(None)
    pooling = int(tbe.pooling_mode)

    def launch_offsets(i):
        v, l, w = batches[i]
        rc = lib.tra_tbe_forward(plan, _lib.ptr(tbe.weights_dev), _lib.ptr(v), _lib.ptr(offs[i]), 0, _lib.ptr(w),
                                 wl["B"], v.numel(), pooling, tbe.output_dtype, _lib.ptr(kout), kout.stride(0), stream)
        if rc != 0:
            _lib.check(rc)

    ws = torch.empty(max(256, lib.tra_tbe_forward_lengths_workspace_bytes(wl["T"], wl["B"], 0)), dtype=torch.uint8, device=dev)

    def launch_lengths(i):
        v, l, w = batches[i]
        rc = lib.tra_tbe_forward_lengths(plan, _lib.ptr(tbe.weights_dev), _lib.ptr(v), _lib.ptr(l), 0, _lib.ptr(w),
                                         wl["B"], wl["T"], v.numel(), pooling, tbe.output_dtype, _lib.ptr(kout),
                                         kout.stride(0), _lib.ptr(ws), stream)
        if rc != 0:
            _lib.check(rc)

    def launch_info(num_keys):
        info = ctypes.create_string_buffer(4096)
        _lib.check(lib.tra_tbe_launch_info(plan, wl["B"], batches[0][0].numel(), pooling, num_keys, info, len(info)))
        return info.value.decode().split("; ")

    def time_launches(fn):
        return time_kernel_launches(fn, args.steps, args.warmup, NB)

    # The module's forward hands a KJT built from lengths to the operator's
    # lengths entry point; when that derives the offsets inside the lookup
    # kernel, that kernel is the one the step runs and the one timed here.
    launches = launch_info(wl["T"]) if wl["pooled"] else launch_info(0)
    fused = any(x.endswith("from_lengths") for x in launches)
    if not fused:
        launches = launch_info(0)
    step_launch = launch_lengths if fused else launch_offsets
    kernel_ms, timed_launches = time_launches(step_launch)
    alg = sum(wl["alg_bytes"][k % args.batches] for k in range(timed_launches)) / timed_launches
    achieved = alg / (kernel_ms * 1e-3) / 1e9
    # spread of single launches: one event pair per launch (includes the launch gap)
    singles = []
    for k in range(min(args.steps, 200)):
        a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a0.record()
        step_launch(k % NB)
        a1.record()
        singles.append((a0, a1))
    torch.cuda.synchronize()
    single_us = sorted(x.elapsed_time(y) * 1e3 for x, y in singles)
    offsets_entry = None
    if fused:
        ms, _ = time_launches(launch_offsets)
        offsets_entry = {
            "kernel_ms": ms, "achieved": alg / (ms * 1e-3) / 1e9, "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "launches_per_call": launch_info(0),
            "note": "the same lookup through tra_tbe_forward with precomputed offsets (the scan is then a separate kernel)",
        }

    # A copy of known size by the library's own copy kernel: hardware-counter
    # runs of this script read FETCH_SIZE / WRITE_SIZE for it next to the lookup.
    cal = torch.empty(2, CAL_COPY_BYTES, dtype=torch.uint8, device=dev)
    cal[0].fill_(1)
    for _ in range(3):
        _lib.check(lib.tra_copy_bytes(_lib.ptr(cal[0]), _lib.ptr(cal[1]), CAL_COPY_BYTES, stream))
    torch.cuda.synchronize()
    del cal

    # HBM traffic per launch is not measured in this run: it comes from the stored
    # hardware-counter profile of the same workload, named here with the commit
    # whose kernels that profile measured (a kernel changed since then makes it stale).
    traffic = None
    traffic_source = None
    tpath = os.path.join(ROOT, "profiles", f"{args.config}_lookup_traffic.json")
    if os.path.exists(tpath):
        try:
            stored = json.load(open(tpath))
            traffic = stored.get("hbm_bytes_per_launch")
            now = kernel_source_hash()
            traffic_source = {
                "file": os.path.relpath(tpath, ROOT),
                "kernel_source_hash_of_profile": stored.get("kernel_source_hash"),
                "kernel_source_hash_now": now,
                # stale: the kernel sources (torchrec_amd/csrc, include) changed since the counters were read
                "stale": stored.get("kernel_source_hash") != now,
                "note": "from the stored rocprofv3 counter runs (FETCH_SIZE, WRITE_SIZE x copy-kernel calibration), not measured in this run",
            }
        except Exception:
            traffic = None

    result = {
        "metric": "pooled lookups/s + achieved HBM GB/s (frac of peak), int4 QuantEBC, 1 GPU",
        "value": total_lookups / el,
        "unit": "lookups/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": el / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": wl["desc"],
            "step": f"QuantEmbeddingBagCollection.forward(KJT) ({args.mode}), {NB} rotating batches",
            "row_alignment": args.row_alignment,
            "row_padding": tbe0.row_padding,
            "row_bytes": sorted(set(tbe0.row_bytes)),
            "row_stride_bytes": sorted(set(tbe0.row_stride)),
            "id_permutation": ("fixed per table" if args.id_permutation == "fixed" else "new per batch (cold head)")
                              if args.config == "c2" else None,
            "rows_total": int(sum(wl["rows"])),
            "store_GB": wl["store_bytes"] / 1e9,
            "lookups_per_step": sum(lookups) / NB,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel": launches[0].split(" ")[0],
            "launches_per_call": launches,
            "kernel_ms": kernel_ms,
            "kernel_launches_timed": timed_launches,
            "kernel_timing": "HIP events around the timed launches, queued behind the untimed ones with no wait in "
                             "between (steady state); at least 500 untimed and 200 timed launches whatever --warmup "
                             "and --steps say",
            "algorithmic_bytes_per_launch": alg,
            "kernel_lookups_per_s": (sum(lookups) / NB) / (kernel_ms * 1e-3),
            "single_launch_us_p50": single_us[len(single_us) // 2],
            "single_launch_us_p90": single_us[int(len(single_us) * 0.9)],
            "offsets_entry": offsets_entry,
        },
    }
    result["host_enqueue_ms_per_step"] = host_ms
    result["pcie_inclusive"] = None if not hsteps else {
        "value": host_lookups / el_host, "unit": "lookups/s", "ms_per_step": el_host / hsteps * 1e3,
        "note": "ids, lengths and weights copied from pinned host memory before every forward; never the headline value",
    }
    if args.request_streams > 1 and wl["pooled"]:
        # Independent requests on separate streams, as a serving loop has them:
        # the first blocks of one lookup start on the CUs that the previous
        # lookup has already left, so its launch and prologue hide behind that
        # lookup's tail.  Kernel durations overlap, so this line carries no
        # per-kernel roofline and is not the headline value.
        ns = args.request_streams
        side = [torch.cuda.Stream() for _ in range(ns)]
        for s_ in side:
            s_.wait_stream(torch.cuda.current_stream())

        def run_streams(steps):
            home = torch.cuda.current_stream()
            try:
                for k in range(steps):
                    torch.cuda.set_stream(side[k % ns])
                    forward(k % NB)
            finally:
                torch.cuda.set_stream(home)

        run_streams(min(args.warmup, 200))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_streams(args.steps)
        torch.cuda.synchronize()
        el_s = time.perf_counter() - t0
        with torch.cuda.stream(side[0]):
            same = bool(torch.equal(out_tensor(forward(0)), out_tensor(outs[0])))
        torch.cuda.synchronize()
        result["concurrent_requests"] = {
            "streams": ns, "value": total_lookups / el_s, "unit": "lookups/s",
            "ms_per_step": el_s / args.steps * 1e3, "algorithmic_GBps": alg / (el_s / args.steps) / 1e9,
            "outputs_equal_single_stream": same,
            "note": f"the same {args.steps} steps dealt round-robin to {ns} HIP streams (independent requests in "
                    "flight); lookups overlap on the GPU, so no per-kernel duration or roofline is quoted here",
        }
    if other:
        result["eager_value"] = total_lookups / el_other
        result["eager_ms_per_step"] = el_other / args.steps * 1e3
    if args.config == "c2" and not args.no_alt_layout and wl["pooled"]:
        other_padding = "none" if tbe0.row_stride != tbe0.row_bytes else "line"
        print(f"[bench] the same workload with row padding '{other_padding}' ...", file=sys.stderr, flush=True)
        result["alt_layout"] = measure_alt_layout(args, dev, other_padding, out_tensor(outs[0]))
    if not args.no_cpu_baseline:
        print("[bench] timing the CPU baseline ...", file=sys.stderr, flush=True)
        result["cpu_baseline"] = cpu_baseline(wl, out_tensor(outs[0]), args.cpu_seconds)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
