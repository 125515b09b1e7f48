"""Benchmark of the weight compress / decompress hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over the whole synthetic weight set: every
weight is quantized + packed (compress), then every packed weight is unpacked +
dequantized (decompress).  Inputs, scales and output buffers are resident in
HBM before the timed region; scales are computed beforehand by the fused
min-max observer (not timed).  Prints ONE JSON line.

Workloads
  llama3-8b-w4a16   (default) 32 x {q,o 4096x4096; k,v 1024x4096; gate,up 14336x4096;
                    down 4096x14336} bf16 N(0, 0.02), symmetric int4, group 128
  w4a16-4096        one 4096 x 4096 weight of the same recipe
"""
import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "compressed-tensors_amd"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak

LLAMA3_8B_LAYER = [
    ("q_proj", 4096, 4096),
    ("k_proj", 1024, 4096),
    ("v_proj", 1024, 4096),
    ("o_proj", 4096, 4096),
    ("gate_proj", 14336, 4096),
    ("up_proj", 14336, 4096),
    ("down_proj", 4096, 14336),
]
GROUP = 128

# HBM bytes per launch of the two fused kernels, averaged over the launches of one
# pass: rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (KiB per dispatch), each scaled
# by what the same counter reads for a plain 1 GiB copy (FETCH_SIZE reads 0.5000 of the
# bytes copied, WRITE_SIZE 1.0000).  The summaries are profiles/pmc_traffic_*.txt.
MEASURED_TRAFFIC = {
    ("llama3-8b-w4a16", "pq_compress_vec_kernel"): 629.1e6,
    ("llama3-8b-w4a16", "pq_decompress_vec_kernel"): 631.1e6,
}


def shapes_for(workload: str):
    if workload == "llama3-8b-w4a16":
        return [(f"layers.{l}.{n}", r, c) for l in range(32) for (n, r, c) in LLAMA3_8B_LAYER]
    if workload == "w4a16-4096":
        return [("w", 4096, 4096)]
    raise SystemExit(f"unknown workload {workload}")


def algorithmic_bytes(shapes):
    """per direction: bf16 dense (2N) + bf16 scales (2G) + packed int4 (N/2)"""
    n = sum(r * c for _, r, c in shapes)
    g = n // GROUP
    return 2 * n + 2 * g + n // 2, n


def cpu_baseline(torch, sample_shapes, seed):
    """the oracle (a step-for-step torch-CPU restatement of the reference's op
    chain) timed on this host's cores, on a bounded sample of the workload"""
    from oracle import pack as opack
    from oracle import quant as oquant

    threads = os.cpu_count() or 1
    threads = min(threads, 16)
    torch.set_num_threads(threads)
    oargs = oquant._Args(num_bits=4, type="int", symmetric=True, strategy="group", group_size=GROUP)
    g = torch.Generator().manual_seed(seed)
    ws = [(torch.randn(r, c, generator=g) * 0.02).bfloat16() for _, r, c in sample_shapes]
    qps = [oquant.observe_weight(w, oargs) for w in ws]
    per_dir, _ = algorithmic_bytes(sample_shapes)
    times = []
    for it in range(4):
        t0 = time.perf_counter()
        for w, (s, z) in zip(ws, qps):
            data = opack.pack_quantized_compress(w, s, oargs, zero_point=z)
            data["weight_scale"] = s
            opack.pack_quantized_decompress(data, oargs)
        dt = time.perf_counter() - t0
        if it:  # first pass is the warm-up
            times.append(dt)
    med = statistics.median(times)
    return {
        "value": 2 * per_dir / med / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": "compress+decompress of " + " + ".join(f"{r}x{c}" for _, r, c in sample_shapes)
        + f" bf16 (W4A16 g128), median of 3 after 1 warm-up, torch {torch.__version__} CPU",
        "seconds": med,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama3-8b-w4a16")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--calib-copies", type=int, default=0,
                    help="launch N plain 1 GiB copies first (byte-counter calibration when profiling)")
    a = ap.parse_args()
    if a.gpus != 1:
        raise SystemExit(
            "bench.py measures one GPU: this path shards by whole tensors with no exchange "
            "step, and no multi-GPU figure is produced (run with --gpus 1)"
        )

    import torch

    from compressed_tensors_amd import _lib
    from compressed_tensors_amd.compressors.pack_quantized import PackedWeightBatch
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    _lib.load()
    dev = torch.device("cuda:0")
    shapes = shapes_for(a.workload)
    args = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group",
                            group_size=GROUP)

    if a.calib_copies:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(a.calib_copies):
            _lib.check(_lib.load().ctmi_calib_copy(src.data_ptr(), dst.data_ptr(), src.numel(),
                                                   _lib.stream_of(dev)))
        torch.cuda.synchronize()
        del src, dst

    # ---- synthetic, seeded inputs resident in HBM
    entries = []
    gen = torch.Generator(device=dev).manual_seed(a.seed)
    for name, r, c in shapes:
        w = (torch.randn(r, c, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
        scale, zp = observe_weight_qparams(w, args)
        entries.append(dict(name=name, weight=w, scale=scale, zero_point=zp,
                            quantization_args=args))
    # The compress side sees the (all-zero, int8) zero points the observer emits, as the
    # reference's state-dict loop passes them on; the decompress side does not, because a
    # symmetric scheme's zero points are not part of the compressed state dict.
    batch = PackedWeightBatch(entries, decompress_zero_points=False)
    per_dir, n_elems = algorithmic_bytes(shapes)
    torch.cuda.synchronize()

    # ---- parity spot check against the oracle (outside the timed region)
    from oracle import pack as opack
    from oracle import quant as oquant

    oargs = oquant._Args(num_bits=4, type="int", symmetric=True, strategy="group", group_size=GROUP)
    batch.compress()
    batch.decompress()
    torch.cuda.synchronize()
    rows = slice(0, 64)
    w0, s0, z0 = (entries[0][k][rows].cpu() for k in ("weight", "scale", "zero_point"))
    want = opack.pack_quantized_compress(w0, s0, oargs, zero_point=z0)
    assert torch.equal(batch.packed[0][rows].cpu(), want["weight_packed"]), "compress parity"
    want_d = opack.pack_quantized_decompress(dict(want, weight_scale=s0), oargs)
    assert torch.equal(batch.dense[0][rows].cpu().view(torch.int16), want_d.view(torch.int16)), \
        "decompress parity"

    # ---- timed region
    for _ in range(a.warmup):
        batch.compress()
        batch.decompress()
    torch.cuda.synchronize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(a.steps)]
    t0 = time.perf_counter()
    for k in range(a.steps):
        ev[k][0].record()
        batch.compress()
        ev[k][1].record()
        batch.decompress()
        ev[k][2].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    comp_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / a.steps
    deco_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / a.steps

    ms_per_step = wall / a.steps * 1e3
    value = 2 * per_dir / (wall / a.steps) / 1e9
    comp_gbs = per_dir / (comp_ms * 1e-3) / 1e9
    deco_gbs = per_dir / (deco_ms * 1e-3) / 1e9
    # the compress kernel does the arithmetic (division, rounding, packing): it is the dominant one
    dom, dom_gbs, dom_ms, n_launch = ("pq_compress_vec_kernel", comp_gbs, comp_ms,
                                      batch.launches(compress=True))
    if deco_ms > comp_ms:
        dom, dom_gbs, dom_ms, n_launch = ("pq_decompress_vec_kernel", deco_gbs, deco_ms,
                                          batch.launches(compress=False))
    traffic = MEASURED_TRAFFIC.get((a.workload, dom))

    out = {
        "metric": "compress+decompress GB/s & % HBM roofline, Llama-3-8B-shaped W4A16 g128",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16->int4 (arithmetic in fp32 rounded to bf16 per op)",
        "data": "synthetic",
        "config": {
            "workload": a.workload,
            "tensors": len(shapes),
            "elements": n_elems,
            "group_size": GROUP,
            "algorithmic_bytes_per_step": 2 * per_dir,
            "scales": "precomputed by the fused min-max observer, outside the timed region",
            "seed": a.seed,
        },
        "hbm_roofline_frac": value / HBM_PEAK_GBS,
        "roofline": {
            "bound": "hbm",
            "kernel": dom,
            "achieved": dom_gbs,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": dom_gbs / HBM_PEAK_GBS,
            "achieved_bytes_per_launch": per_dir / n_launch,
            "traffic": traffic,
            "traffic_unit": "HBM bytes per launch (FETCH_SIZE + WRITE_SIZE, copy-calibrated)",
            "avg_launch_ms": dom_ms / n_launch,
            "launches_per_step": n_launch,
            "compress_GBs": comp_gbs,
            "decompress_GBs": deco_gbs,
            "compress_ms": comp_ms,
            "decompress_ms": deco_ms,
        },
        "parity": "bit-exact vs oracle on the first 64 rows of tensor 0 (checked before timing)",
    }
    if not a.no_cpu_baseline:
        sample = LLAMA3_8B_LAYER  # one layer of 32; the other 31 are identical work
        if a.workload == "w4a16-4096":
            sample = [("w", 4096, 4096)]
        out["cpu_baseline"] = cpu_baseline(torch, sample, a.seed)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
