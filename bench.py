"""Benchmark of the weight compress / decompress hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over the whole synthetic weight set: every
weight is quantized + packed (compress), then every packed weight is unpacked +
dequantized (decompress).  Inputs, scales and output buffers are resident in
HBM before the timed region; scales are computed beforehand by the fused
min-max observer (not timed).  Prints ONE JSON line.

With no --workload the line is the headline (llama3-8b-w4a16) and carries, under
"configs", a short run of every other configuration below (its operations, the
roofline fraction of its dominant kernel, MFMA utilisation for the Hadamard
kernels, its own CPU baseline) and, under "api_level", ModelCompressor.compress_model
/ decompress_model timed on a 224-Linear module tree of the same shapes.
--only-headline leaves those out.

Workloads
  llama3-8b-w4a16   (default) 32 x {q,o 4096x4096; k,v 1024x4096; gate,up 14336x4096;
                    down 4096x14336} bf16 N(0, 0.02), symmetric int4, group 128
  w4a16-4096        one 4096 x 4096 weight of the same recipe
The other configurations of the same path, each a list of operations timed one
by one (HIP events on the launch stream) over rotating copies of the inputs, so
that no pass finds its input in the last-level cache:
  fp8-w8a8          per-channel fp8 weights of the same 224 shapes (0.1 % outliers x20)
                    + dynamic per-token fp8 activation quantization, 8192 x 4096
  sparse            sparse-bitmask on a 50 % pruned 8192 x 8192 bf16 weight; sparse-24-bitmask
                    on a 2:4 pruned, fp8-quantized 14336 x 4096 weight
  nvfp4             nvfp4-pack-quantized on 14336 x 4096 and 4096 x 14336 bf16 weights
                    + dynamic nvfp4 activation quantization, 4096 x 4096
  one-shot          the default set with no scales given: min-max observer, qparams,
                    quantize and pack, as separate passes and as one
  hadamard          block-128 and full 4096 rotations of 8192 x 4096 activations and of
                    4096 x 4096 / 14336 x 4096 weights
  standalone        single reference functions called on their own, one call per 14336 x 4096
                    tensor: round_to_quantized_type, pack_to_int32 / unpack_from_int32,
                    pack_fp4_to_uint8 / unpack_fp4_from_uint8, get_24_bytemasks
  api               ModelCompressor.compress_model / decompress_model on a module tree of the
                    default set's 224 weights (wall time of the host mirror above the C ABI)
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

PROFILES = ROOT / "profiles"
MFMA_BF16_PEAK = 2.5e15  # dense bf16 MFMA, published peak


def measured_traffic(workload, kernel, operation=None):
    """HBM bytes per launch from the committed counter summaries: lines of the form
    `traffic_bytes_per_launch <workload> <kernel> <bytes> [op=<operation>]` in
    profiles/*pmc_traffic*.txt (rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE, KiB per
    dispatch, each scaled by what the same counter reads for a plain 1 GiB copy).  A line
    that names the operation (counters of a run with --only-op) wins over one for the kernel
    alone; where a kernel has lines with operations and none of them is this one, nothing is
    returned (another operation's launches move other bytes).
    -> (bytes or None, file name or None)"""
    by_kernel, tagged = None, False
    for path in sorted(PROFILES.glob("*pmc_traffic*.txt")):
        for line in path.read_text().splitlines():
            f = line.split(None, 4)
            if len(f) < 4 or f[0] != "traffic_bytes_per_launch" or f[1] != workload or f[2] != kernel:
                continue
            if len(f) == 5:
                tagged = True
                if operation is not None and f[4].strip() == "op=" + operation:
                    return float(f[3]), f"profiles/{path.name}"
            elif by_kernel is None:
                by_kernel = (float(f[3]), f"profiles/{path.name}")
    if by_kernel is not None and not tagged:
        return by_kernel
    return None, None


def cpu_threads():
    """threads the CPU baseline runs on: every core this process may use (its affinity
    mask, capped by OMP_NUM_THREADS where the host sets one for its share of the machine)"""
    n = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cap = os.environ.get("OMP_NUM_THREADS", "")
    if cap.isdigit() and int(cap) > 0:
        n = min(n, int(cap))
    return max(n, 1)


def median_time(run, repeats=5):
    """median of `repeats` timed runs after one warm-up"""
    times = []
    for it in range(repeats + 1):
        t0 = time.perf_counter()
        run()
        dt = time.perf_counter() - t0
        if it:
            times.append(dt)
    return statistics.median(times)


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

    threads = cpu_threads()
    torch.set_num_threads(threads)
    oargs = oquant._Args(num_bits=4, type="int", symmetric=True, strategy="group", group_size=GROUP)
    g = torch.Generator().manual_seed(seed)
    ws = [(torch.randn(r, c, generator=g) * 0.02).bfloat16() for _, r, c in sample_shapes]
    qps = [oquant.observe_weight(w, oargs) for w in ws]
    per_dir, _ = algorithmic_bytes(sample_shapes)

    def run():
        for w, (s, z) in zip(ws, qps):
            data = opack.pack_quantized_compress(w, s, oargs, zero_point=z)
            data["weight_scale"] = s
            opack.pack_quantized_decompress(data, oargs)

    med = median_time(run)
    return {
        "value": 2 * per_dir / med / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "host_cpu_count": os.cpu_count(),
        "kind": "port",
        "sample": "compress+decompress of " + " + ".join(f"{r}x{c}" for _, r, c in sample_shapes)
        + f" bf16 (W4A16 g128), median of 5 after 1 warm-up, torch {torch.__version__} CPU",
        "sample_short": f"compress+decompress of {len(sample_shapes)} of the workload's tensors "
                        f"({sum(r * c for _, r, c in sample_shapes)} elements), median of 5",
        "seconds": med,
    }


# ---------------------------------------------------------------------------------------------
# The other configurations: lists of operations on the C ABI, prepared once and timed one by one
def chained(n_tensors, per_launch=8):
    """kernel launches of a many-tensor entry point: every chain kernel of the library takes up
    to 8 tensors a launch"""
    return -(-n_tensors // per_launch)


class Op:
    """primary=False: an operation that is only there to be compared with (the separate steps a
    fused operation replaces, one call per weight against one call for all)"""

    def __init__(self, name, calls, nbytes, kernel, primary=True, mfma_flops=None, launches=None,
                 useful_flops=None, passes_bytes=None):
        self.name, self.calls, self.nbytes, self.kernel = name, calls, nbytes, kernel
        self.primary = primary
        self.mfma_flops = mfma_flops  # flops the kernel issues on the matrix cores, per pass
        # ... and those of them the transform needs: an fp32 operand that goes into a product as
        # three bf16 terms is issued three times and needed once
        self.useful_flops = mfma_flops if useful_flops is None else useful_flops
        # launches of `kernel` per pass: one per call unless a call chains several
        self.launches = len(calls) if launches is None else launches
        # bytes the operation has to move when its result needs more than one pass over the
        # input (sparse-bitmask compression: the values' positions depend on a prefix sum over
        # the whole tensor, so the tensor is read once for the mask and counts and once more
        # to be compacted): the floor of the method, next to the format's algorithmic bytes
        self.passes_bytes = passes_bytes
        self.ms = 0.0


def time_ops(torch, ops, steps, warmup):
    """every op is a list of enqueue closures (one per rotating input copy); per-op GPU time from
    events recorded on the launch stream around each op"""
    def one_pass(record):
        marks = []
        for op in ops:
            if record:
                e = torch.cuda.Event(enable_timing=True); e.record(); marks.append(e)
            for call in op.calls:
                call()
        if record:
            e = torch.cuda.Event(enable_timing=True); e.record(); marks.append(e)
        return marks
    for _ in range(warmup):
        one_pass(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    all_marks = [one_pass(True) for _ in range(steps)]
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    for i, op in enumerate(ops):
        op.ms = sum(m[i].elapsed_time(m[i + 1]) for m in all_marks) / steps
    return wall / steps


def other_workload(torch, name, seed):
    """-> (metric, ops, keep-alive list)"""
    import ctypes
    from compressed_tensors_amd import _lib
    from compressed_tensors_amd.quantization import (QuantizationArgs, compute_dynamic_scales_and_zp,
                                                     generate_gparam, observe_weight_qparams)
    from compressed_tensors_amd.quantization.forward import build_qparams
    from compressed_tensors_amd.transform.hadamard import deterministic_hadamard_matrix

    lib = _lib.load()
    dev = torch.device("cuda:0")
    st = _lib.stream_of(dev)
    code = _lib.dtype_code
    gen = torch.Generator(device=dev).manual_seed(seed)
    keep = []
    FP8 = torch.float8_e4m3fn

    def randn(r, c, std=1.0):
        return (torch.randn(r, c, generator=gen, device=dev) * std).to(torch.bfloat16)

    def qdq(x, out, plan, do_q, do_dq):
        keep.extend([x, out, plan])
        rows = x.numel() // x.shape[-1]
        args = (x.data_ptr(), code(x.dtype), out.data_ptr(), code(out.dtype), rows, x.shape[-1],
                ctypes.byref(plan.qp), do_q, do_dq, st)
        return lambda: _lib.check(lib.ctmi_qdq(*args))

    def observe(x, blk_cols, args, scale, zp, gscale=None):
        keep.extend([x, scale, zp, gscale])
        rows = x.numel() // x.shape[-1]
        qtype = _lib.QTYPE_FLOAT if args.type == "float" else _lib.QTYPE_INT
        a = (x.data_ptr(), code(x.dtype), rows, x.shape[-1], blk_cols, qtype, args.num_bits,
             int(args.symmetric), _lib.ptr(gscale), scale.data_ptr(), code(scale.dtype),
             zp.data_ptr(), code(zp.dtype), None, None, st)
        return lambda: _lib.check(lib.ctmi_observe_qparams(*a))

    def observe_many(items, args):
        """items: (x, blk_cols, scale, zp): one ctmi_observe_qparams_many call for the list"""
        jobs = (_lib.ObserveJob * len(items))()
        for j, (x, blk_cols, scale, zp) in zip(jobs, items):
            j.x, j.scale, j.zero_point, j.global_scale = x.data_ptr(), scale.data_ptr(), zp.data_ptr(), None
            j.rows, j.cols, j.blk_cols, j.x_dtype = x.numel() // x.shape[-1], x.shape[-1], blk_cols, code(x.dtype)
        keep.extend([jobs, items])
        qtype = _lib.QTYPE_FLOAT if args.type == "float" else _lib.QTYPE_INT
        a = (jobs, len(items), qtype, args.num_bits, int(args.symmetric), -1, code(items[0][3].dtype), st)
        return lambda: _lib.check(lib.ctmi_observe_qparams_many(*a))

    def dynamic(x, out, blk_cols, args, gscale=None):
        keep.extend([x, out, gscale])
        rows = x.numel() // x.shape[-1]
        qtype = _lib.QTYPE_FLOAT if args.type == "float" else _lib.QTYPE_INT
        fp4 = args.num_bits == 4 and args.type == "float"
        a = (x.data_ptr(), code(x.dtype), out.data_ptr(), rows, x.shape[-1], blk_cols, qtype,
             args.num_bits, int(args.symmetric), _lib.ptr(gscale), None,
             code(FP8 if fp4 else x.dtype), None, code(FP8 if args.type == "float" else torch.int8), st)
        return lambda: _lib.check(lib.ctmi_dynamic_qdq(*a))

    if name == "fp8-w8a8":
        args = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="channel")
        from compressed_tensors_amd.compressors import QuantizedWeightBatch
        entries, n = [], 0
        for _, r, c in shapes_for("llama3-8b-w4a16"):
            w = randn(r, c, 0.02)
            hot = torch.rand(r, c, generator=gen, device=dev) < 1e-3
            w = torch.where(hot, w * 20, w)
            scale, zp = observe_weight_qparams(w, args)
            entries.append(dict(weight=w, scale=scale, zero_point=None, quantization_args=args, observed_zp=zp))
            n += r * c
        batch = QuantizedWeightBatch(entries)   # one ctmi_qdq_many call per direction
        keep.append(batch)
        q_calls, d_calls = [batch.compress], [batch.decompress]
        # one-shot: scales + fp8 codes from one pass over weights that have no scales yet,
        # against the observer and the quantizer one after the other (one call per weight each)
        w_obs, w_q, w_one = [], [], []
        w_obs_many = [observe_many([(e["weight"], e["weight"].shape[1], e["scale"], e["observed_zp"])
                                    for e in entries], args)]
        for e, codes in zip(entries, batch.codes):
            w, sc = e["weight"], e["scale"]
            r, c = w.shape
            w_obs.append(observe(w, c, args, sc, e["observed_zp"]))
            w_q.append(qdq(w, codes, build_qparams(w, sc, None, args), 1, 0))
            oa = (w.data_ptr(), code(w.dtype), codes.data_ptr(), r, c, c, 1, 8, 1, sc.data_ptr(), code(sc.dtype),
                  None, code(FP8), st)
            w_one.append(lambda oa=oa: _lib.check(lib.ctmi_observe_quantize(*oa)))
        oq_jobs = (_lib.ObserveQuantizeJob * len(entries))()
        for job, e, codes in zip(oq_jobs, entries, batch.codes):
            w, sc = e["weight"], e["scale"]
            job.x, job.codes, job.scale, job.zero_point = w.data_ptr(), codes.data_ptr(), sc.data_ptr(), None
            job.rows, job.cols, job.blk_cols, job.x_dtype = w.shape[0], w.shape[1], w.shape[1], code(w.dtype)
        keep.append(oq_jobs)
        om = (oq_jobs, len(entries), 1, 8, 1, -1, code(FP8), st)
        w_many = [lambda om=om: _lib.check(lib.ctmi_observe_quantize_many(*om))]
        # block strategy (128 x 128 cells): the same one pass, a block per workgroup
        w_blk, blk_scales = [], []
        for e, codes in zip(entries, batch.codes):
            w = e["weight"]
            r, c = w.shape
            sb = torch.empty(r // 128, c // 128, dtype=w.dtype, device=dev)
            blk_scales.append(sb)
            ob = (w.data_ptr(), code(w.dtype), codes.data_ptr(), r, c, 128, 128, 1, 8, 1, sb.data_ptr(),
                  code(sb.dtype), None, code(FP8), st)
            w_blk.append(lambda ob=ob: _lib.check(lib.ctmi_observe_quantize_blocks(*ob)))
        bjobs = (_lib.ObserveQuantizeBlocksJob * len(entries))()
        for job, e, codes, sb in zip(bjobs, entries, batch.codes, blk_scales):
            w = e["weight"]
            job.x, job.codes, job.scale, job.zero_point = w.data_ptr(), codes.data_ptr(), sb.data_ptr(), None
            job.rows, job.cols, job.blk_rows, job.blk_cols = w.shape[0], w.shape[1], 128, 128
            job.x_dtype = code(w.dtype)
        keep.append(bjobs)
        bm = (bjobs, len(entries), 1, 8, 1, -1, code(FP8), st)
        w_blk_many = [lambda bm=bm: _lib.check(lib.ctmi_observe_quantize_blocks_many(*bm))]
        keep.append(blk_scales)
        acts, a_obs, a_fq, a_dyn = [], [], [], []
        targs = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="token",
                                 dynamic=True)
        for _ in range(8):  # 8 x 67 MB: more than the last-level cache
            x = randn(8192, 4096)
            x[:, torch.rand(4096, generator=gen, device=dev) < 5e-3] *= 50
            x = x.reshape(1, 8192, 4096)
            s, z = compute_dynamic_scales_and_zp(x, targs)
            out = torch.empty_like(x)
            a_obs.append(observe(x, 4096, targs, s, z))
            a_fq.append(qdq(x, out, build_qparams(x, s, z, targs), 1, 1))
            a_dyn.append(dynamic(x, out, 4096, targs))
            acts.append(x)
        na = 8 * 8192 * 4096
        ops = [Op("weights: quantize to fp8, per channel (224 tensors)", q_calls, 3 * n, "qdq_vec_many_kernel", launches=chained(len(entries))),
               Op("weights: dequantize from fp8 (224 tensors)", d_calls, 3 * n, "qdq_vec_many_kernel", launches=chained(len(entries))),
               Op("weights one-shot: per-channel observer (224 calls)", w_obs, 2 * n, "observe_wide_kernel", primary=False),
               Op("weights one-shot: per-channel observer, one call (8 per launch)", w_obs_many, 2 * n,
                  "observe_wide_chain_kernel", launches=chained(len(entries))),
               Op("weights one-shot: quantize with those scales (224 calls)", w_q, 3 * n, "qdq_vec_kernel", primary=False),
               Op("weights one-shot: scales + fp8 codes in one pass (224 calls)", w_one, 3 * n, "dynamic_rows_kernel", primary=False),
               Op("weights one-shot: scales + fp8 codes in one pass, one call (8 per launch)", w_many, 3 * n, "dynamic_rows_many_kernel", launches=chained(len(entries))),
               Op("weights one-shot, 128x128 blocks: scales + fp8 codes in one pass (224 calls)", w_blk, 3 * n,
                  "observe_quantize_blocks_kernel", primary=False),
               Op("weights one-shot, 128x128 blocks: scales + fp8 codes in one pass, one call (8 per launch)", w_blk_many,
                  3 * n, "observe_quantize_blocks_many_kernel", launches=chained(len(entries))),
               Op("activations: per-token min-max + scales (8 x 8192x4096)", a_obs, 2 * na, "observe_wide_kernel"),
               Op("activations: per-token fp8 fake-quantize (8 x 8192x4096)", a_fq, 4 * na, "qdq_vec_kernel"),
               Op("activations: scales + fake-quantize in one pass (8 x 8192x4096)", a_dyn, 4 * na, "dynamic_rows_kernel")]
        return "fp8 W8A8 quantize/dequantize GB/s, Llama-3-8B-shaped weights + per-token activations", ops, keep

    if name == "sparse":
        copies = 6
        c_calls, d_calls, s_calls, t_calls, two_step, one_step = [], [], [], [], [], []
        back_two, back_one, s16_calls, t16_calls, pk_calls, up_calls = [], [], [], [], [], []
        stacked_jobs = []
        nb = 8192 * 8192
        nnz_total = 0
        for _ in range(copies):
            w = randn(8192, 8192, 0.02)
            thr = w.float().abs().flatten().kthvalue(nb // 2).values
            w = torch.where(w.float().abs() <= thr, torch.zeros_like(w), w)
            rows, cols = w.shape
            bitmask = torch.empty(rows, cols // 8, dtype=torch.uint8, device=dev)
            offs = torch.empty(rows, dtype=torch.int64, device=dev)
            total = torch.empty(1, dtype=torch.int64, device=dev)
            tmp = torch.empty(lib.ctmi_bitmask_tmp_bytes(rows, cols), dtype=torch.uint8, device=dev)
            a = (w.data_ptr(), 2, 1, bitmask.data_ptr(), offs.data_ptr(), total.data_ptr(), tmp.data_ptr(), rows, cols, st)
            _lib.check(lib.ctmi_bitmask_count(*a))
            nnz = int(total.item())
            nnz_total += nnz
            values = torch.empty(nnz, dtype=torch.bfloat16, device=dev)
            b = (w.data_ptr(), 2, bitmask.data_ptr(), offs.data_ptr(), values.data_ptr(), rows, cols, st)
            dense = torch.empty_like(w)
            d = (values.data_ptr(), nnz, 2, bitmask.data_ptr(), None, dense.data_ptr(), tmp.data_ptr(), rows, cols, st)
            keep.extend([w, bitmask, offs, total, tmp, values, dense])
            c_calls.append(lambda a=a, b=b: (_lib.check(lib.ctmi_bitmask_count(*a)), _lib.check(lib.ctmi_bitmask_compact(*b))))
            d_calls.append(lambda d=d: _lib.check(lib.ctmi_bitmask_decompress(*d)))
        n24 = 14336 * 4096
        cargs = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="channel")
        from compressed_tensors_amd.compressors import get_24_bytemasks
        from compressed_tensors_amd.quantization import quantize
        copies24 = 16  # values + bitmask of the codes are 37 MB a copy: well beyond the 256 MB last-level cache
        s24_jobs, s24_jobs16 = [], []
        for _ in range(copies24):
            w = randn(14336, 4096, 0.02)
            w = torch.where(get_24_bytemasks(w), w, torch.zeros_like(w))
            scale, _ = observe_weight_qparams(w, cargs)
            q = quantize(w, scale, None, cargs, dtype=FP8)
            rows, cols = q.shape
            values = torch.empty(rows, cols // 2, dtype=FP8, device=dev)
            bitmask = torch.empty(rows, cols // 8, dtype=torch.uint8, device=dev)
            dense = torch.empty_like(q)
            tmp = torch.empty(lib.ctmi_sparse24_tmp_bytes(rows, cols, 1), dtype=torch.uint8, device=dev)
            a = (q.data_ptr(), code(FP8), values.data_ptr(), bitmask.data_ptr(), rows, cols, st)
            d = (values.data_ptr(), values.numel(), 1, bitmask.data_ptr(), dense.data_ptr(), tmp.data_ptr(), rows, cols, st)
            _lib.check(lib.ctmi_sparse24_compress(*a))
            keep.extend([q, values, bitmask, dense, tmp])
            s_calls.append(lambda a=a: _lib.check(lib.ctmi_sparse24_compress(*a)))
            # the stacked case: bf16 -> fp8 codes -> 2:4, two steps against one
            plan = build_qparams(w, scale, None, cargs)
            keep.extend([w, scale, plan])
            qa = (w.data_ptr(), code(w.dtype), q.data_ptr(), code(q.dtype), rows, cols, ctypes.byref(plan.qp), 1, 0, st)
            fa = (w.data_ptr(), code(w.dtype), values.data_ptr(), bitmask.data_ptr(), rows, cols, ctypes.byref(plan.qp), st)
            two_step.append(lambda qa=qa, a=a: (_lib.check(lib.ctmi_qdq(*qa)), _lib.check(lib.ctmi_sparse24_compress(*a))))
            one_step.append(lambda fa=fa: _lib.check(lib.ctmi_quantize_sparse24_compress(*fa)))
            t_calls.append(lambda d=d: _lib.check(lib.ctmi_sparse24_decompress(*d)))
            s24_jobs.append((q, values, bitmask, dense, rows, cols))
            # the bool mask of the weight <-> its packed form
            bools = get_24_bytemasks(w)
            bools_back = torch.empty_like(bools)
            packed = torch.empty(rows, cols // 8, dtype=torch.uint8, device=dev)
            keep.extend([bools, bools_back, packed])
            pk = (bools.data_ptr(), packed.data_ptr(), rows, cols, st)
            up = (packed.data_ptr(), bools_back.data_ptr(), rows, cols, st)
            _lib.check(lib.ctmi_pack_bitmasks(*pk))
            pk_calls.append(lambda pk=pk: _lib.check(lib.ctmi_pack_bitmasks(*pk)))
            up_calls.append(lambda up=up: _lib.check(lib.ctmi_unpack_bitmasks(*up)))
            # the same format on the bf16 weight itself (a sparse-only checkpoint)
            values16 = torch.empty(rows, cols // 2, dtype=w.dtype, device=dev)
            dense16 = torch.empty_like(w)
            tmp16 = torch.empty(lib.ctmi_sparse24_tmp_bytes(rows, cols, 2), dtype=torch.uint8, device=dev)
            bitmask16 = torch.empty_like(bitmask)
            keep.extend([values16, dense16, tmp16, bitmask16])
            a16 = (w.data_ptr(), code(w.dtype), values16.data_ptr(), bitmask16.data_ptr(), rows, cols, st)
            d16 = (values16.data_ptr(), values16.numel(), 2, bitmask16.data_ptr(), dense16.data_ptr(), tmp16.data_ptr(), rows, cols, st)
            _lib.check(lib.ctmi_sparse24_compress(*a16))
            s24_jobs16.append((w, values16, bitmask16, dense16, rows, cols))
            s16_calls.append(lambda a16=a16: _lib.check(lib.ctmi_sparse24_compress(*a16)))
            t16_calls.append(lambda d16=d16: _lib.check(lib.ctmi_sparse24_decompress(*d16)))
            # ... and the way back: 2:4 -> fp8 codes -> bf16
            back = torch.empty_like(w)
            tmp_dq = torch.empty(lib.ctmi_sparse24_dequantize_tmp_bytes(rows, cols), dtype=torch.uint8, device=dev)
            keep.extend([back, tmp_dq])
            dq = (dense.data_ptr(), code(dense.dtype), back.data_ptr(), code(back.dtype), rows, cols, ctypes.byref(plan.qp), 0, 1, st)
            fd = (values.data_ptr(), values.numel(), code(FP8), bitmask.data_ptr(), back.data_ptr(), code(back.dtype),
                  tmp_dq.data_ptr(), rows, cols, ctypes.byref(plan.qp), st)
            back_two.append(lambda d=d, dq=dq: (_lib.check(lib.ctmi_sparse24_decompress(*d)), _lib.check(lib.ctmi_qdq(*dq))))
            back_one.append(lambda fd=fd: _lib.check(lib.ctmi_sparse24_decompress_dequantize(*fd)))
            stacked_jobs.append((w, values, bitmask, back, rows, cols, plan))
        # the stacked case for all weights from one call (8 per launch)
        qc, qd = (_lib.Stacked24Job * copies24)(), (_lib.Stacked24Job * copies24)()
        for k, (w, values, bitmask, back, rows, cols, plan) in enumerate(stacked_jobs):
            for job, dense_side in ((qc[k], w), (qd[k], back)):
                job.dense, job.values, job.bitmask = dense_side.data_ptr(), values.data_ptr(), bitmask.data_ptr()
                job.rows, job.cols = rows, cols
                job.dense_dtype, job.values_dtype, job.qp = code(dense_side.dtype), code(FP8), plan.qp
        qcm, qdm = (qc, copies24, st), (qd, copies24, st)
        keep.extend([qc, qd])
        cj, dj = (_lib.Sparse24Job * copies24)(), (_lib.Sparse24Job * copies24)()
        for k, (q, values, bitmask, dense, rows, cols) in enumerate(s24_jobs):
            for job, full in ((cj[k], q), (dj[k], dense)):
                job.dense, job.values, job.bitmask = full.data_ptr(), values.data_ptr(), bitmask.data_ptr()
                job.nvalues, job.rows, job.cols = values.numel(), rows, cols
        cj16, dj16 = (_lib.Sparse24Job * copies24)(), (_lib.Sparse24Job * copies24)()
        for k, (w, values, bitmask, dense, rows, cols) in enumerate(s24_jobs16):
            for job, full in ((cj16[k], w), (dj16[k], dense)):
                job.dense, job.values, job.bitmask = full.data_ptr(), values.data_ptr(), bitmask.data_ptr()
                job.nvalues, job.rows, job.cols = values.numel(), rows, cols
        keep.extend([cj, dj, cj16, dj16])
        cm = (cj, copies24, code(FP8), st)
        dm = (dj, copies24, 1, st)
        cm16 = (cj16, copies24, code(s24_jobs16[0][0].dtype), st)
        dm16 = (dj16, copies24, 2, st)
        bm_bytes = copies * (2 * nb + nb // 8 + 8 * 8192) + 2 * nnz_total
        s24_bytes = copies24 * (n24 + n24 // 2 + n24 // 8)
        fused24_bytes = copies24 * (2 * n24 + n24 // 2 + n24 // 8)  # what the one-pass form has to move
        # two passes over the dense tensor: (dense in, bitmask + counts out), a scan of the counts,
        # (dense + bitmask + offsets in, values out)
        bm_passes = copies * (2 * 2 * nb + 2 * (nb // 8) + 3 * 8 * 8192) + 2 * nnz_total
        ops = [Op("sparse-bitmask compress, 8192x8192 bf16, 50 % zeros (mask+offsets, then compaction)", c_calls, bm_bytes,
                  "bitmask_compact_rows_kernel", passes_bytes=bm_passes),
               Op("sparse-bitmask decompress (positions from the bitmask alone)", d_calls, bm_bytes, "bitmask_scatter_tiles_kernel"),
               Op("sparse-24-bitmask compress, 14336x4096 fp8", s_calls, s24_bytes, "sparse24_compress_kernel"),
               Op("sparse-24-bitmask decompress", t_calls, s24_bytes, "sparse24_scatter_kernel"),
               Op("sparse-24-bitmask compress, fp8, all 16 in one call (8 per launch)",
                  [lambda: _lib.check(lib.ctmi_sparse24_compress_many(*cm))], s24_bytes, "sparse24_compress_chain_kernel", launches=chained(copies24)),
               Op("sparse-24-bitmask decompress, fp8, all 16 in one call (8 per launch)",
                  [lambda: _lib.check(lib.ctmi_sparse24_decompress_many(*dm))], s24_bytes, "sparse24_scatter_kernel", launches=chained(copies24)),
               Op("sparse-24-bitmask compress, 14336x4096 bf16", s16_calls, 2 * s24_bytes - copies24 * (n24 // 8), "sparse24_compress_kernel"),
               Op("sparse-24-bitmask decompress, bf16", t16_calls, 2 * s24_bytes - copies24 * (n24 // 8), "sparse24_scatter_kernel"),
               Op("sparse-24-bitmask compress, bf16, all 16 in one call (8 per launch)",
                  [lambda: _lib.check(lib.ctmi_sparse24_compress_many(*cm16))],
                  2 * s24_bytes - copies24 * (n24 // 8), "sparse24_compress_chain_kernel", launches=chained(copies24)),
               Op("sparse-24-bitmask decompress, bf16, all 16 in one call (8 per launch)",
                  [lambda: _lib.check(lib.ctmi_sparse24_decompress_many(*dm16))],
                  2 * s24_bytes - copies24 * (n24 // 8), "sparse24_scatter_kernel", launches=chained(copies24)),
               Op("pack_bitmasks, 14336x4096 bool", pk_calls, copies24 * (n24 + n24 // 8), "pack_bitmasks"),
               Op("unpack_bitmasks", up_calls, copies24 * (n24 + n24 // 8), "unpack_bitmasks"),
               Op("bf16 -> fp8 codes -> 2:4 compress, two steps (14336x4096)", two_step, fused24_bytes, "qdq_vec_kernel", primary=False),
               Op("bf16 -> fp8 codes -> 2:4 compress, one pass", one_step, fused24_bytes, "quant_sparse24_compress_kernel"),
               Op("2:4 decompress -> fp8 codes -> bf16, two steps", back_two, fused24_bytes, "qdq_vec_kernel", primary=False),
               Op("2:4 decompress -> fp8 codes -> bf16, one pass", back_one, fused24_bytes, "sparse24_scatter_dequant_kernel"),
               Op("bf16 -> fp8 codes -> 2:4 compress, one pass, all 16 in one call (8 per launch)",
                  [lambda: _lib.check(lib.ctmi_quantize_sparse24_compress_many(*qcm))], fused24_bytes,
                  "quant_sparse24_compress_chain_kernel", launches=chained(copies24)),
               Op("2:4 decompress -> fp8 codes -> bf16, one pass, all 16 in one call (8 per launch)",
                  [lambda: _lib.check(lib.ctmi_sparse24_decompress_dequantize_many(*qdm))], fused24_bytes,
                  "sparse24_scatter_dequant_chain_kernel", launches=chained(copies24))]
        return "sparse-bitmask / sparse-24-bitmask compress+decompress GB/s", ops, keep

    if name == "nvfp4":
        args = QuantizationArgs(num_bits=4, type="float", symmetric=True, strategy="tensor_group",
                                group_size=16)
        ops = []
        for r, c in ((14336, 4096), (4096, 14336)):
            c_calls, d_calls, many_c, many_d = [], [], [], []
            n_copies = 16  # the packed side (33 MB a copy) has to exceed the 256 MB last-level cache too
            for _ in range(n_copies):
                w = randn(r, c, 0.02)
                gs = generate_gparam(w.min().reshape(1), w.max().reshape(1))
                scale, zp = observe_weight_qparams(w, args, global_scale=gs)
                packed = torch.empty(r, c // 2, dtype=torch.uint8, device=dev)
                dense = torch.empty_like(w)
                cp = build_qparams(w, scale, zp, args, None, gs)
                dp = build_qparams(w, scale, None, args, None, gs)
                keep.extend([w, gs, scale, zp, packed, dense, cp, dp])
                ca = (w.data_ptr(), code(w.dtype), packed.data_ptr(), r, c, ctypes.byref(cp.qp), st)
                da = (packed.data_ptr(), dense.data_ptr(), code(dense.dtype), r, c, ctypes.byref(dp.qp), st)
                c_calls.append(lambda ca=ca: _lib.check(lib.ctmi_nvfp4_compress(*ca)))
                d_calls.append(lambda da=da: _lib.check(lib.ctmi_nvfp4_decompress(*da)))
                many_c.append((w.data_ptr(), packed.data_ptr(), code(w.dtype), cp))
                many_d.append((packed.data_ptr(), dense.data_ptr(), code(dense.dtype), dp))
            nbytes = n_copies * (2 * r * c + r * c // 16 + r * c // 2)
            ops += [Op(f"nvfp4 compress {r}x{c} (x{n_copies})", c_calls, nbytes, "nvfp4_compress_vec_kernel"),
                    Op(f"nvfp4 decompress {r}x{c} (x{n_copies})", d_calls, nbytes, "nvfp4_decompress_vec_kernel")]
            # the same tensors through the multi-weight entry points (what the compressor's
            # state-dict path calls): 8 per launch
            for many, entry, kernel, what in ((many_c, lib.ctmi_nvfp4_compress_many, "nvfp4_compress_chain_kernel", "compress"),
                                              (many_d, lib.ctmi_nvfp4_decompress_many, "nvfp4_decompress_chain_kernel", "decompress")):
                jobs = (_lib.WeightJob * len(many))()
                for job, (src, dst, dt, plan) in zip(jobs, many):
                    job.src, job.dst, job.rows, job.cols, job.dense_dtype, job.qp = src, dst, r, c, dt, plan.qp
                keep.append(jobs)
                m = (jobs, len(many), st)
                ops.append(Op(f"nvfp4 {what} {r}x{c} (x{n_copies}), one call (8 per launch)",
                              [lambda m=m, entry=entry: _lib.check(entry(*m))], nbytes, kernel, launches=chained(n_copies)))
        # the Llama-3-8B-shaped set: one call per weight against all 224 in one call
        from compressed_tensors_amd.compressors import Fp4WeightBatch
        entries, single_c, single_d, n_set = [], [], [], 0
        for _, r, c in shapes_for("llama3-8b-w4a16"):
            w = randn(r, c, 0.02)
            gs = generate_gparam(w.min().reshape(1), w.max().reshape(1))
            scale, zp = observe_weight_qparams(w, args, global_scale=gs)
            entries.append(dict(weight=w, scale=scale, global_scale=gs, quantization_args=args))
            n_set += r * c
        batch = Fp4WeightBatch(entries)
        batch.dense  # allocate the decompress side now: its addresses go into the per-weight calls
        keep.append(batch)
        for i in range(batch.n):
            cj, dj = batch._cjobs[i], batch._djobs[i]
            ca = (cj.src, cj.dense_dtype, cj.dst, cj.rows, cj.cols, ctypes.byref(cj.qp), st)
            da = (dj.src, dj.dst, dj.dense_dtype, dj.rows, dj.cols, ctypes.byref(dj.qp), st)
            single_c.append(lambda ca=ca: _lib.check(lib.ctmi_nvfp4_compress(*ca)))
            single_d.append(lambda da=da: _lib.check(lib.ctmi_nvfp4_decompress(*da)))
        set_bytes = 2 * n_set + n_set // 16 + n_set // 2
        ops += [Op("nvfp4 compress, Llama-3-8B set, one call per weight (224)", single_c, set_bytes, "nvfp4_compress_vec_kernel", primary=False),
                Op("nvfp4 compress, Llama-3-8B set, all weights in one call (8 per launch)", [batch.compress], set_bytes, "nvfp4_compress_chain_kernel", launches=chained(batch.n)),
                Op("nvfp4 decompress, Llama-3-8B set, one call per weight (224)", single_d, set_bytes, "nvfp4_decompress_vec_kernel", primary=False),
                Op("nvfp4 decompress, Llama-3-8B set, all weights in one call (8 per launch)", [batch.decompress], set_bytes, "nvfp4_decompress_chain_kernel", launches=chained(batch.n))]
        # one-shot: group scales + codes from one pass over weights whose global scale is known
        oj = (_lib.ObserveNvfp4Job * batch.n)()
        one_calls = []
        for i, e in enumerate(entries):
            w, gs = e["weight"], e["global_scale"]
            r, c = w.shape
            sc_out = torch.empty(r, c // 16, dtype=FP8, device=dev)
            keep.append(sc_out)
            cj = batch._cjobs[i]
            oj[i].x, oj[i].global_scale, oj[i].packed, oj[i].scale = w.data_ptr(), gs.data_ptr(), cj.dst, sc_out.data_ptr()
            oj[i].rows, oj[i].cols, oj[i].x_dtype = r, c, code(w.dtype)
            oa = (w.data_ptr(), code(w.dtype), r, c, gs.data_ptr(), cj.dst, sc_out.data_ptr(), st)
            one_calls.append(lambda oa=oa: _lib.check(lib.ctmi_observe_nvfp4_compress(*oa)))
        keep.append(oj)
        om = (oj, batch.n, st)
        ops += [Op("nvfp4 one-shot (scales + codes), Llama-3-8B set, one call per weight (224)", one_calls, set_bytes,
                   "nvfp4_observe_compress_kernel", primary=False),
                Op("nvfp4 one-shot (scales + codes), Llama-3-8B set, all weights in one call (8 per launch)",
                   [lambda: _lib.check(lib.ctmi_observe_nvfp4_compress_many(*om))], set_bytes,
                   "nvfp4_observe_compress_chain_kernel", launches=chained(batch.n))]
        aargs = QuantizationArgs(num_bits=4, type="float", symmetric=True, strategy="tensor_group",
                                 group_size=16, dynamic="local")
        o_calls, f_calls, y_calls = [], [], []
        for _ in range(16):
            x = randn(4096, 4096)
            gs = generate_gparam(x.min().reshape(1), x.max().reshape(1))
            s, z = compute_dynamic_scales_and_zp(x, aargs, None, global_scale=gs)
            out = torch.empty_like(x)
            o_calls.append(observe(x, 16, aargs, s, z, gs))
            f_calls.append(qdq(x, out, build_qparams(x, s, None, aargs, None, gs), 1, 1))
            y_calls.append(dynamic(x, out, 16, aargs, gs))
        na = 16 * 4096 * 4096
        ops += [Op("nvfp4 activations: group-16 scales (16 x 4096x4096)", o_calls, 2 * na + na // 16, "observe_flat_kernel"),
                Op("nvfp4 activations: fake-quantize (16 x 4096x4096)", f_calls, 4 * na + na // 16, "nvfp4_qdq_vec_kernel"),
                Op("nvfp4 activations: scales + fake-quantize in one pass (16 x 4096x4096)", y_calls, 4 * na, "nvfp4_dynamic_kernel")]
        return "nvfp4-pack-quantized compress/decompress + activation fake-quantize GB/s", ops, keep

    if name == "one-shot":
        # the Llama-3-8B-shaped set, no scales yet: observer + qparams + quantize + pack
        args = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group", group_size=GROUP)
        sep_obs, sep_cmp, fused, job_fields, n, keep2, obs_zps = [], [], [], [], 0, [], []
        for _, r, c in shapes_for("llama3-8b-w4a16"):
            w = randn(r, c, 0.02)
            scale, zp = observe_weight_qparams(w, args)
            packed = torch.empty(r, c // 8, dtype=torch.int32, device=dev)
            plan = build_qparams(w, scale, None, args, None, None)
            keep.extend([w, scale, zp, packed, plan])
            keep2.append((w, scale, packed))
            obs_zps.append(zp)
            sep_obs.append(observe(w, GROUP, args, scale, zp))
            ca = (w.data_ptr(), code(w.dtype), packed.data_ptr(), r, c, ctypes.byref(plan.qp), st)
            sep_cmp.append(lambda ca=ca: _lib.check(lib.ctmi_pack_quantized_compress(*ca)))
            fa = (w.data_ptr(), code(w.dtype), r, c, GROUP, 4, 1, packed.data_ptr(), scale.data_ptr(), None, st)
            fused.append(lambda fa=fa: _lib.check(lib.ctmi_observe_pack_quantized(*fa)))
            job_fields.append((w.data_ptr(), packed.data_ptr(), scale.data_ptr(), None, r, c, GROUP,
                               code(w.dtype), 4, 1))
            n += r * c
        jobs = (_lib.ObservePackJob * len(job_fields))()
        for j, f in zip(jobs, job_fields):
            (j.x, j.packed, j.scale, j.zero_point, j.rows, j.cols, j.blk_cols, j.x_dtype,
             j.num_bits, j.symmetric) = f
        keep.append(jobs)
        many = [lambda: _lib.check(lib.ctmi_observe_pack_quantized_many(jobs, len(job_fields), st))]
        sep_obs_many = [observe_many([(w, GROUP, scale, zp) for (w, scale, _), zp in zip(keep2, obs_zps)], args)]
        # the same set with activation ordering (one random g_idx per row length): the group of
        # a column is looked up, min / max meet in LDS
        from compressed_tensors_amd.quantization.forward import _column_groups
        col_groups, gidx_one, gidx_cmp = {}, [], []
        for (w, scale, packed) in list(keep2):
            r, c = w.shape
            if c not in col_groups:
                perm = torch.randperm(c, generator=torch.Generator().manual_seed(seed + c)).to(dev)
                col_groups[c] = ((perm // GROUP).to(torch.int32), _column_groups((perm // GROUP).to(torch.int32), GROUP))
            g_idx, cg = col_groups[c]
            ga = (w.data_ptr(), code(w.dtype), r, c, GROUP, 4, 1, cg.data_ptr(), packed.data_ptr(),
                  scale.data_ptr(), None, st)
            gidx_one.append(lambda ga=ga: _lib.check(lib.ctmi_observe_pack_quantized_gidx(*ga)))
            gplan = build_qparams(w, scale, None, args, g_idx, None)
            keep2.append(gplan)
            gc = (w.data_ptr(), code(w.dtype), packed.data_ptr(), r, c, ctypes.byref(gplan.qp), st)
            gidx_cmp.append(lambda gc=gc: _lib.check(lib.ctmi_pack_quantized_compress(*gc)))
        keep.extend(keep2)
        keep.append(col_groups)
        g = n // GROUP
        ops = [Op("observer + qparams, group 128 (224 tensors, one call each)", sep_obs, 2 * n + 3 * g, "observe_flat_kernel", primary=False),
               Op("observer + qparams, group 128, all 224 tensors in one call (8 per launch)", sep_obs_many, 2 * n + 3 * g,
                  "observe_flat_chain_kernel", launches=chained(len(job_fields))),
               Op("quantize + pack with those scales (one call each)", sep_cmp, 2 * n + 2 * g + n // 2, "pq_compress_vec_kernel", primary=False),
               Op("observer + qparams + quantize + pack in one pass (one call each)", fused, 2 * n + 2 * g + n // 2, "observe_pack_groups_kernel", primary=False),
               Op("the same, all 224 tensors in one call (8 per launch)", many, 2 * n + 2 * g + n // 2, "observe_pack_groups_kernel", launches=chained(len(job_fields))),
               Op("activation ordering (g_idx): quantize + pack with given scales, the second of two passes (one call each)",
                  gidx_cmp, 2 * n + 2 * g + n // 2, "pq_gidx_compress_kernel", primary=False),
               Op("activation ordering (g_idx): observer + qparams + quantize + pack in one pass (one call each)",
                  gidx_one, 2 * n + 2 * g + n // 2, "observe_pack_table_kernel", primary=False)]
        return "one-shot W4A16 g128 compression GB/s (no scales given), Llama-3-8B-shaped weights", ops, keep

    if name == "standalone":
        # the entry points of single reference functions called on their own (a caller that
        # holds codes, a mask or a tensor to round already): one call per 14336x4096 tensor
        ops = []
        # A8 on its own: every element to the nearest fp8 value, dtype kept
        r_calls, nr = [], 0
        for _ in range(8):
            x = randn(14336, 4096)
            out = torch.empty_like(x)
            keep.extend([x, out])
            ra = (x.data_ptr(), out.data_ptr(), code(x.dtype), x.numel(), 1, 8, st)
            r_calls.append(lambda ra=ra: _lib.check(lib.ctmi_round_to_quantized_type(*ra)))
            nr += x.numel()
        ops.append(Op("round_to_quantized_type alone (fp8), bf16 14336x4096 (x8)", r_calls, 4 * nr, "round_to_type_kernel"))
        # A9 / A10 on their own: int8 codes <-> packed words (callers that hold codes already)
        pk_calls, up_calls, n_codes = [], [], 0
        for _ in range(16):
            r, c = 14336, 4096
            codes = torch.randint(-8, 8, (r, c), generator=gen, device=dev, dtype=torch.int8)
            words = torch.empty(r, c // 8, dtype=torch.int32, device=dev)
            back = torch.empty_like(codes)
            keep.extend([codes, words, back])
            pa = (codes.data_ptr(), words.data_ptr(), r, c, 4, 1, st)
            ua = (words.data_ptr(), back.data_ptr(), r, c, 4, 1, st)
            _lib.check(lib.ctmi_pack_to_int32(*pa))
            pk_calls.append(lambda pa=pa: _lib.check(lib.ctmi_pack_to_int32(*pa)))
            up_calls.append(lambda ua=ua: _lib.check(lib.ctmi_unpack_from_int32(*ua)))
            n_codes += r * c
        ops += [Op("pack_to_int32 alone: int8 codes -> 4-bit words, 14336x4096 (x16)", pk_calls, n_codes + n_codes // 2,
                   "pack_dim1_vec_kernel"),
                Op("unpack_from_int32 alone, 14336x4096 (x16)", up_calls, n_codes + n_codes // 2,
                   "unpack_dim1_vec_kernel")]
        # A13 / A14 on their own: values already on the e2m1 grid <-> two codes a byte
        grid = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], device=dev)
        p4_calls, u4_calls, n4 = [], [], 0
        for _ in range(16):
            r, c = 14336, 4096
            x = (grid[torch.randint(0, 8, (r, c), generator=gen, device=dev)]
                 * (torch.randint(0, 2, (r, c), generator=gen, device=dev) * 2 - 1)).to(torch.bfloat16)
            codes = torch.empty(r, c // 2, dtype=torch.uint8, device=dev)
            back = torch.empty_like(x)
            keep.extend([x, codes, back])
            pa = (x.data_ptr(), code(x.dtype), codes.data_ptr(), r, c, st)
            ua = (codes.data_ptr(), back.data_ptr(), code(back.dtype), r, c, st)
            _lib.check(lib.ctmi_pack_fp4_to_uint8(*pa))
            p4_calls.append(lambda pa=pa: _lib.check(lib.ctmi_pack_fp4_to_uint8(*pa)))
            u4_calls.append(lambda ua=ua: _lib.check(lib.ctmi_unpack_fp4_from_uint8(*ua)))
            n4 += r * c
        ops += [Op("pack_fp4_to_uint8 alone, bf16 14336x4096 (x16)", p4_calls, 2 * n4 + n4 // 2, "fp4_pack_vec_kernel"),
                Op("unpack_fp4_from_uint8 alone, to bf16 (x16)", u4_calls, 2 * n4 + n4 // 2, "fp4_unpack_vec_kernel")]
        # A20 on its own: the top-2-of-4 mask of a dense tensor, one bool per element
        bm_calls, nbm = [], 0
        for _ in range(8):
            w = randn(14336, 4096, 0.02)
            mask = torch.empty(w.shape, dtype=torch.bool, device=dev)
            keep.extend([w, mask])
            bm = (w.data_ptr(), code(w.dtype), mask.data_ptr(), w.numel(), st)
            bm_calls.append(lambda bm=bm: _lib.check(lib.ctmi_get_24_bytemasks(*bm)))
            nbm += w.numel()
        ops.append(Op("get_24_bytemasks alone, bf16 14336x4096 -> bool (x8)", bm_calls, 3 * nbm, "bytemask24_vec_kernel"))
        return "single reference functions called on their own, GB/s", ops, keep

    if name == "hadamard":
        ops = []
        tensors = {"activations 8192x4096 (x8)": [randn(8192, 4096) for _ in range(8)],
                   "weights 4096x4096 (x16)": [randn(4096, 4096, 0.02) for _ in range(16)],
                   "weights 14336x4096 (x5)": [randn(14336, 4096, 0.02) for _ in range(5)]}
        for n, (a_dim, b_dim) in ((128, (1, 128)), (4096, (64, 64))):
            q = (torch.randint(0, 2, (n,), generator=torch.Generator().manual_seed(seed)) * 2 - 1).float().to(dev)
            mb = deterministic_hadamard_matrix(b_dim, torch.bfloat16, dev).contiguous()
            ma = deterministic_hadamard_matrix(a_dim, torch.bfloat16, dev).contiguous() if a_dim > 1 else None
            keep.extend([q, mb, ma])
            # size 128: no matrix argument stands for Sylvester's matrix (the kernel that keeps none
            # in memory); the kernel that is handed the matrix is timed beside it on one line
            mbp = None if a_dim == 1 else mb.data_ptr()
            rows_kernel = "sylvester128_quant_pack_kernel" if a_dim == 1 else "hadamard_kron_kernel"
            for label, xs in tensors.items():
                calls, with_matrix = [], []
                for x in xs:
                    out = torch.empty_like(x)
                    keep.extend([x, out])
                    a = (x.data_ptr(), out.data_ptr(), code(x.dtype), x.numel(), a_dim, b_dim,
                         _lib.ptr(ma), mbp, q.data_ptr(), None, st)
                    calls.append(lambda a=a: _lib.check(lib.ctmi_hadamard_apply(*a)))
                    am = a[:7] + (mb.data_ptr(),) + a[8:]
                    with_matrix.append(lambda am=am: _lib.check(lib.ctmi_hadamard_apply(*am)))
                nb = sum(4 * x.numel() for x in xs)
                # matrix-core flops per element: 2 b for the one product of a block-b rotation;
                # 2 b + 3 * 2 a for a Kronecker pair (the fp32 result of the first product goes
                # into the second as three bf16 terms)
                per_elem = 2 * b_dim if a_dim == 1 else 2 * b_dim + 6 * a_dim
                flops = sum(per_elem * x.numel() for x in xs)
                useful = sum(2 * (a_dim + b_dim if a_dim > 1 else b_dim) * x.numel() for x in xs)
                # size 4096 on the matrix cores: kept to compare with the butterfly kernel below,
                # which is what hadamard_apply picks for this size
                ops.append(Op(f"random-sign Hadamard, size {n}{' (matrix cores)' if a_dim > 1 else ''}: {label}",
                              calls, nb, rows_kernel,
                              primary=a_dim == 1 and not label.startswith("weights 4096x4096"), mfma_flops=flops,
                              useful_flops=useful))
                if a_dim == 1 and label.startswith("weights 14336x4096"):
                    ops.append(Op(f"random-sign Hadamard, size {n}, any matrix of 128 (passed as an argument): {label}",
                                  with_matrix, nb, "hadamard_rows_kernel", primary=False, mfma_flops=flops,
                                  useful_flops=useful))
                if label.startswith("weights 4096x4096"):
                    jobs = (_lib.HadamardJob * len(xs))()
                    outs = [torch.empty_like(x) for x in xs]
                    for job, x, out in zip(jobs, xs, outs):
                        job.x, job.out, job.numel = x.data_ptr(), out.data_ptr(), x.numel()
                    keep.extend([jobs, outs])
                    m = (jobs, len(xs), code(xs[0].dtype), a_dim, b_dim, _lib.ptr(ma), mbp,
                         q.data_ptr(), None, st)
                    ops.append(Op(f"random-sign Hadamard, size {n}{' (matrix cores)' if a_dim > 1 else ''}: {label}, "
                                  "one call (8 per launch)",
                                  [lambda m=m: _lib.check(lib.ctmi_hadamard_apply_many(*m))], nb,
                                  rows_kernel,
                                  primary=a_dim == 1, mfma_flops=flops, useful_flops=useful,
                                  launches=chained(len(xs))))
        # sizes 4096 and 8192 as butterflies in registers (ctmi_sylvester_apply_many): what
        # hadamard_apply and HadamardTransform.forward run for these sizes
        tensors["activations 4096x8192 (x8)"] = [randn(4096, 8192) for _ in range(8)]
        for n, labels in ((4096, ("activations 8192x4096 (x8)", "weights 4096x4096 (x16)", "weights 14336x4096 (x5)")),
                          (8192, ("activations 4096x8192 (x8)",))):
            q = (torch.randint(0, 2, (n,), generator=torch.Generator().manual_seed(seed)) * 2 - 1).float().to(dev)
            keep.append(q)
            for label in labels:
                xs = tensors[label]
                calls = []
                many = (_lib.HadamardJob * len(xs))()
                for i, x in enumerate(xs):
                    out = torch.empty_like(x)
                    one = (_lib.HadamardJob * 1)()
                    for job in (one[0], many[i]):
                        job.x, job.out, job.numel = x.data_ptr(), out.data_ptr(), x.numel()
                    keep.extend([x, out, one])
                    a = (one, 1, code(x.dtype), n, q.data_ptr(), None, st)
                    calls.append(lambda a=a: _lib.check(lib.ctmi_sylvester_apply_many(*a)))
                keep.append(many)
                nb = sum(4 * x.numel() for x in xs)
                # bf16 runs of 4096 go to the kernel that does the 64 x 64 factor over the inner
                # index as ONE exact bf16 product on the matrix cores (2 * 64 flops an element, all
                # of them needed) and the other factor as butterflies; 8192 is butterflies only
                kernel = "fwht_mfma_kernel" if n == 4096 else "fwht_lds_kernel"
                flops = sum(2 * 64 * x.numel() for x in xs) if n == 4096 else None
                ops.append(Op(f"random-sign Hadamard, size {n}: {label}", calls, nb, kernel,
                              primary=n == 4096 and not label.startswith("weights 4096x4096"), mfma_flops=flops))
                if label.startswith("weights 4096x4096"):
                    m = (many, len(xs), code(xs[0].dtype), n, q.data_ptr(), None, st)
                    ops.append(Op(f"random-sign Hadamard, size {n}: {label}, one call (8 per launch)",
                                  [lambda m=m: _lib.check(lib.ctmi_sylvester_apply_many(*m))], nb, kernel,
                                  mfma_flops=flops, launches=chained(len(xs))))
        # 14336 = 224 x 64: a known Hadamard matrix of order 224 (here: any +-1 matrix, the kernel's
        # work does not depend on the entries) times Sylvester(64), as the reference builds the
        # rotation in front of Llama-3's down projections
        xs14 = [randn(4096, 14336) for _ in range(5)]
        ma224 = (torch.randint(0, 2, (224, 224), generator=torch.Generator().manual_seed(seed)) * 2 - 1
                 ).bfloat16().to(dev).contiguous()
        mb64 = deterministic_hadamard_matrix(64, torch.bfloat16, dev).contiguous()
        q14 = (torch.randint(0, 2, (14336,), generator=torch.Generator().manual_seed(seed)) * 2 - 1).float().to(dev)
        keep.extend([ma224, mb64, q14])
        calls = []
        for x in xs14:
            out = torch.empty_like(x)
            keep.extend([x, out])
            a = (x.data_ptr(), out.data_ptr(), code(x.dtype), x.numel(), 224, 64, ma224.data_ptr(),
                 mb64.data_ptr(), q14.data_ptr(), None, st)
            calls.append(lambda a=a: _lib.check(lib.ctmi_hadamard_apply(*a)))
        ops.append(Op("random-sign Hadamard, size 14336 = 224 x 64, both factors as matrix products: "
                      "activations 4096x14336 (x5)", calls,
                      sum(4 * x.numel() for x in xs14), "hadamard_kron_kernel", primary=False,
                      mfma_flops=sum((2 * 64 + 6 * 224) * x.numel() for x in xs14),
                      useful_flops=sum(2 * (64 + 224) * x.numel() for x in xs14)))
        # the same transform as HadamardTransform.forward runs it: the block on the matrix cores,
        # Sylvester(64) as butterflies (no matrix for it: mb_t = NULL)
        calls = []
        for x in xs14:
            out = torch.empty_like(x)
            keep.append(out)
            a = (x.data_ptr(), out.data_ptr(), code(x.dtype), x.numel(), 224, 64, ma224.data_ptr(),
                 None, q14.data_ptr(), None, st)
            calls.append(lambda a=a: _lib.check(lib.ctmi_hadamard_apply(*a)))
        # (sizes beyond the benchmark's configuration, block 128 and full 4096: listed, not part of
        # the configuration's aggregate)
        ops.append(Op("random-sign Hadamard, size 14336 = 224 x 64: activations 4096x14336 (x5)", calls,
                      sum(4 * x.numel() for x in xs14), "block_sylvester64_kernel", primary=False,
                      mfma_flops=sum(2 * 224 * x.numel() for x in xs14)))
        # 3584 = 224 x 16 (the reference takes the largest block of its table: hidden sizes such
        # as 3584 and 3072 come out as a large block times a short Sylvester factor): four runs
        # share the kernel's 64 columns
        xs35 = [randn(16384, 3584) for _ in range(5)]
        q35 = (torch.randint(0, 2, (3584,), generator=torch.Generator().manual_seed(seed)) * 2 - 1).float().to(dev)
        keep.append(q35)
        calls = []
        for x in xs35:
            out = torch.empty_like(x)
            keep.extend([x, out])
            a = (x.data_ptr(), out.data_ptr(), code(x.dtype), x.numel(), 224, 16, ma224.data_ptr(),
                 None, q35.data_ptr(), None, st)
            calls.append(lambda a=a: _lib.check(lib.ctmi_hadamard_apply(*a)))
        ops.append(Op("random-sign Hadamard, size 3584 = 224 x 16: activations 16384x3584 (x5)", calls,
                      sum(4 * x.numel() for x in xs35), "block_sylvester64_kernel", primary=False,
                      mfma_flops=sum(2 * 224 * x.numel() for x in xs35)))
        # rotation (block 128) + symmetric int4 group-128 quantization + pack_to_int32, one pass
        mb = deterministic_hadamard_matrix(128, torch.bfloat16, dev).contiguous()
        q = (torch.randint(0, 2, (128,), generator=torch.Generator().manual_seed(seed)) * 2 - 1).float().to(dev)
        keep.extend([mb, q])
        for label in ("weights 4096x4096 (x16)", "weights 14336x4096 (x5)"):
            calls, calls_matrix = [], []
            for x in tensors[label]:
                packed = torch.empty(x.shape[0], x.shape[1] // 8, dtype=torch.int32, device=dev)
                scale = torch.empty(x.shape[0], x.shape[1] // 128, dtype=torch.bfloat16, device=dev)
                keep.extend([packed, scale])
                # no matrix argument: Sylvester's matrix of 128, what hadamard_quantize_pack passes
                # for the reference's own matrices of this size
                a = (x.data_ptr(), code(x.dtype), x.numel(), 128, None, q.data_ptr(), None,
                     4, 1, packed.data_ptr(), scale.data_ptr(), None, st)
                calls.append(lambda a=a: _lib.check(lib.ctmi_hadamard_quant_pack(*a)))
                ax = a[:4] + (mb.data_ptr(),) + a[5:]
                calls_matrix.append(lambda ax=ax: _lib.check(lib.ctmi_hadamard_quant_pack(*ax)))
            nb = sum(2 * x.numel() + x.numel() // 2 + 2 * x.numel() // 128 for x in tensors[label])
            flops = sum(2 * 128 * x.numel() for x in tensors[label])
            ops.append(Op(f"fused: Hadamard 128 + int4 g128 quantize + pack, {label}", calls, nb,
                          "sylvester128_quant_pack_kernel", primary=not label.startswith("weights 4096x4096"),
                          mfma_flops=flops))
            if not label.startswith("weights 4096x4096"):
                ops.append(Op(f"fused: any 128 x 128 matrix + int4 g128 quantize + pack, {label}", calls_matrix, nb,
                              "hadamard_quant_pack_kernel", primary=False, mfma_flops=flops))
            if label.startswith("weights 4096x4096"):
                xs = tensors[label]
                jobs = (_lib.HadamardPackJob * len(xs))()
                for job, x in zip(jobs, xs):
                    packed = torch.empty(x.shape[0], x.shape[1] // 8, dtype=torch.int32, device=dev)
                    scale = torch.empty(x.shape[0], x.shape[1] // 128, dtype=torch.bfloat16, device=dev)
                    keep.extend([packed, scale])
                    job.x, job.packed, job.scale, job.rotated, job.numel = (
                        x.data_ptr(), packed.data_ptr(), scale.data_ptr(), None, x.numel())
                keep.append(jobs)
                m = (jobs, len(xs), code(xs[0].dtype), 128, None, q.data_ptr(), None, 4, 1, st)
                ops.append(Op(f"fused: Hadamard 128 + int4 g128 quantize + pack, {label}, one call (8 per launch)",
                              [lambda m=m: _lib.check(lib.ctmi_hadamard_quant_pack_many(*m))], nb,
                              "sylvester128_quant_pack_kernel", mfma_flops=flops, launches=chained(len(xs))))
        # the full 4096-wide rotation (64 x 64) with the same quantization in its epilogue
        mb64 = deterministic_hadamard_matrix(64, torch.bfloat16, dev).contiguous()
        q4k = (torch.randint(0, 2, (4096,), generator=torch.Generator().manual_seed(seed)) * 2 - 1).float().to(dev)
        keep.extend([mb64, q4k])
        for label in ("weights 4096x4096 (x16)", "weights 14336x4096 (x5)"):
            xs = tensors[label]
            calls = []
            many = (_lib.HadamardPackJob * len(xs))()
            for i, x in enumerate(xs):
                one = (_lib.HadamardPackJob * 1)()
                for job in (one[0], many[i]):
                    packed = torch.empty(x.shape[0], x.shape[1] // 8, dtype=torch.int32, device=dev)
                    scale = torch.empty(x.shape[0], x.shape[1] // 128, dtype=torch.bfloat16, device=dev)
                    keep.extend([packed, scale])
                    job.x, job.packed, job.scale, job.rotated, job.numel = (
                        x.data_ptr(), packed.data_ptr(), scale.data_ptr(), None, x.numel())
                keep.append(one)
                a = (one, 1, code(x.dtype), 64, 64, mb64.data_ptr(), mb64.data_ptr(), q4k.data_ptr(), None,
                     128, 4, 1, st)
                calls.append(lambda a=a: _lib.check(lib.ctmi_hadamard_kron_quant_pack_many(*a)))
            keep.append(many)
            nb = sum(2 * x.numel() + x.numel() // 2 + 2 * x.numel() // 128 for x in xs)
            flops = sum((2 * 64 + 6 * 64) * x.numel() for x in xs)
            useful = sum(2 * (64 + 64) * x.numel() for x in xs)
            ops.append(Op(f"fused: Hadamard 4096 (matrix cores) + int4 g128 quantize + pack, {label}", calls, nb,
                          "hadamard_kron_kernel", primary=False, mfma_flops=flops, useful_flops=useful))
            if label.startswith("weights 4096x4096"):
                m = (many, len(xs), code(xs[0].dtype), 64, 64, mb64.data_ptr(), mb64.data_ptr(),
                     q4k.data_ptr(), None, 128, 4, 1, st)
                ops.append(Op(f"fused: Hadamard 4096 (matrix cores) + int4 g128 quantize + pack, {label}, "
                              "one call (8 per launch)",
                              [lambda m=m: _lib.check(lib.ctmi_hadamard_kron_quant_pack_many(*m))], nb,
                              "hadamard_kron_kernel", primary=False, mfma_flops=flops, useful_flops=useful,
                              launches=chained(len(xs))))
            # the same through the butterfly kernel (what hadamard_quantize_pack picks)
            calls = []
            for i in range(len(xs)):
                one = (_lib.HadamardPackJob * 1)()
                one[0] = many[i]
                keep.append(one)
                a = (one, 1, code(xs[i].dtype), 4096, q4k.data_ptr(), None, 128, 4, 1, st)
                calls.append(lambda a=a: _lib.check(lib.ctmi_sylvester_quant_pack_many(*a)))
            flops = sum(2 * 64 * x.numel() for x in xs)
            ops.append(Op(f"fused: Hadamard 4096 + int4 g128 quantize + pack, {label}", calls, nb,
                          "fwht_mfma_kernel", primary=not label.startswith("weights 4096x4096"), mfma_flops=flops))
            if label.startswith("weights 4096x4096"):
                m = (many, len(xs), code(xs[0].dtype), 4096, q4k.data_ptr(), None, 128, 4, 1, st)
                ops.append(Op(f"fused: Hadamard 4096 + int4 g128 quantize + pack, {label}, one call (8 per launch)",
                              [lambda m=m: _lib.check(lib.ctmi_sylvester_quant_pack_many(*m))], nb,
                              "fwht_mfma_kernel", mfma_flops=flops, launches=chained(len(xs))))
        return "Hadamard rotation GB/s, block 128 (bf16 MFMA) and full 4096 / 8192 (butterflies), and fused with int4 packing", ops, keep

    raise SystemExit(f"unknown workload {name}")


def cpu_baseline_other(torch, workload, seed):
    """the oracle's restatement of one representative operation pair of the workload, timed on
    this host's cores on a bounded sample (same definition of algorithmic bytes as the GPU line)"""
    from oracle import hadamard as ohad
    from oracle import pack as opack
    from oracle import quant as oquant
    from oracle import sparse as osparse

    threads = cpu_threads()
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(seed)
    if workload == "fp8-w8a8":
        spec = dict(num_bits=8, type="float", symmetric=True, strategy="channel")
        oargs = oquant._Args(**spec)
        w = (torch.randn(14336, 4096, generator=g) * 0.02).bfloat16()
        s, z = oquant.observe_weight(w, oargs)
        nbytes, what = 6 * w.numel(), "fp8 per-channel quantize + dequantize of a 14336x4096 bf16 weight"

        def run():
            codes = opack.naive_compress(w, s, oargs, zero_point=z)
            opack.naive_decompress({"weight": codes, "weight_scale": s})
    elif workload == "sparse":
        w = (torch.randn(8192, 8192, generator=g) * 0.02).bfloat16()
        w[torch.rand(8192, 8192, generator=g) < 0.5] = 0
        nnz = int((w != 0).sum())
        nbytes = 2 * (2 * w.numel() + w.numel() // 8 + 2 * nnz) + 8 * 8192
        what = "sparse-bitmask compress + decompress of a 8192x8192 bf16 tensor, half zeros"

        def run():
            values, bitmask, _ = osparse.bitmask_compress(w)
            osparse.bitmask_decompress(values, bitmask, list(w.shape))
    elif workload == "nvfp4":
        spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
        oargs = oquant._Args(**spec)
        w = (torch.randn(14336, 4096, generator=g) * 0.02).bfloat16()
        gs = oquant.generate_gparam(*[t.reshape(1) for t in torch.aminmax(w)])
        s, z = oquant.observe_weight(w, oargs, global_scale=gs)
        n = w.numel()
        nbytes, what = 2 * (2 * n + n // 16 + n // 2), "nvfp4 compress + decompress of a 14336x4096 bf16 weight"

        def run():
            packed = opack.nvfp4_compress(w, s, gs, oargs)
            opack.nvfp4_decompress(packed, s, gs)
    elif workload == "hadamard":
        x = torch.randn(8192, 4096, generator=g).bfloat16()
        q = (torch.randint(0, 2, (128,), generator=g) * 2 - 1).double()
        weight = q[:, None] * ohad.deterministic_hadamard_matrix(128, torch.float64)
        nbytes, what = 4 * x.numel(), "random-sign Hadamard of size 128 on a 8192x4096 bf16 activation (fp64 matmul, as the reference's offline precision)"

        def run():
            ohad.hadamard_forward(weight, x, "input")
    elif workload == "one-shot":
        spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=GROUP)
        oargs = oquant._Args(**spec)
        w = (torch.randn(14336, 4096, generator=g) * 0.02).bfloat16()
        n = w.numel()
        nbytes, what = 2 * n + 2 * n // GROUP + n // 2, "observer + qparams + quantize + pack of a 14336x4096 bf16 weight (W4A16 g128)"

        def run():
            s, z = oquant.observe_weight(w, oargs)
            opack.pack_quantized_compress(w, s, oargs, zero_point=z)
    elif workload == "standalone":
        codes = torch.randint(-8, 8, (14336, 4096), generator=g, dtype=torch.int8)
        n = codes.numel()
        nbytes, what = 2 * (n + n // 2), "pack_to_int32 + unpack_from_int32 of 14336x4096 int8 codes (4 bits)"

        def run():
            opack.unpack_from_int32(opack.pack_to_int32(codes, 4), 4, codes.shape)
    else:
        return None
    med = median_time(run)
    return {"value": nbytes / med / 1e9, "unit": "GB/s", "cores": threads,
            "host_cpu_count": os.cpu_count(), "kind": "port",
            "sample": what + f", median of 5 after 1 warm-up, torch {torch.__version__} CPU",
            "seconds": med}


def run_other(torch, workload, seed, steps, warmup, with_cpu_baseline=True, only_op=None):
    """one of the other configurations -> its result object (same fields as the headline
    line, plus the per-operation table).  only_op: time just the operations whose name contains
    this text, or equals it after a leading "=" (a counter run then sees the launches of that operation and no others)"""
    metric, ops, keep = other_workload(torch, workload, seed)
    if only_op:
        exact = only_op.startswith("=")
        ops = [op for op in ops if (op.name == only_op[1:] if exact else only_op in op.name)]
        if not ops:
            raise SystemExit(f"no operation of {workload} is named like {only_op!r}")
        for op in ops:
            op.primary = True
    step_s = time_ops(torch, ops, steps, warmup)
    total_bytes = sum(op.nbytes for op in ops)
    gpu_ms = sum(op.ms for op in ops)
    # the roofline object describes the operation most of the time goes to (comparison-only
    # operations aside); every operation's own rate is in `operations`
    slow = max((op for op in ops if op.primary), key=lambda op: op.ms)
    n_launch = slow.launches
    traffic, traffic_source = measured_traffic(workload, slow.kernel, slow.name)

    def op_row(op):
        row = {"name": op.name, "kernel": op.kernel, "GBs": op.nbytes / (op.ms * 1e-3) / 1e9,
               "frac_of_hbm_peak": op.nbytes / (op.ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
               "ms": op.ms, "algorithmic_bytes": op.nbytes,
               "for_comparison_only": not op.primary}
        row["launches"] = op.launches
        if op.passes_bytes is not None:
            row["bytes_of_its_passes"] = op.passes_bytes
            row["frac_of_hbm_peak_on_bytes_of_its_passes"] = op.passes_bytes / (op.ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        if op.mfma_flops is not None:
            row["mfma_TFLOPs"] = op.mfma_flops / (op.ms * 1e-3) / 1e12
            row["mfma_utilisation"] = op.mfma_flops / (op.ms * 1e-3) / MFMA_BF16_PEAK
            row["mfma_utilisation_useful_flops"] = op.useful_flops / (op.ms * 1e-3) / MFMA_BF16_PEAK
        return row

    out = {
        "metric": metric,
        "value": total_bytes / (gpu_ms * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": step_s * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 (codes as the format says; arithmetic in the dtype the reference's chain promotes to)",
        "data": "synthetic",
        "config": {"workload": workload, "seed": seed,
                   "value_is": "algorithmic bytes of all operations / sum of their GPU times",
                   "value_without_comparison_lines_is": "the same over the operations the library's own "
                                                        "dispatch runs (for_comparison_only false)"},
        "value_without_comparison_lines": sum(op.nbytes for op in ops if op.primary) /
                                          (sum(op.ms for op in ops if op.primary) * 1e-3) / 1e9,
        "roofline": {"bound": "hbm", "kernel": slow.kernel, "operation": slow.name,
                     "achieved": slow.nbytes / (slow.ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": slow.nbytes / (slow.ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "achieved_bytes_per_launch": slow.nbytes / n_launch,
                     "traffic": traffic, "traffic_source": traffic_source,
                     "avg_launch_ms": slow.ms / n_launch, "launches_per_step": n_launch},
        "operations": [op_row(op) for op in ops],
        "ms_per_step_gpu": gpu_ms,
    }
    mfma = [op for op in ops if op.mfma_flops is not None and op.primary]
    if mfma:
        best = max(mfma, key=lambda op: op.mfma_flops / op.ms)
        out["mfma_utilisation"] = {
            "peak": "2.5 PFLOP/s dense bf16", "kernel": best.kernel, "operation": best.name,
            "achieved_TFLOPs": best.mfma_flops / (best.ms * 1e-3) / 1e12,
            "frac": best.mfma_flops / (best.ms * 1e-3) / MFMA_BF16_PEAK,
            "frac_useful_flops": best.useful_flops / (best.ms * 1e-3) / MFMA_BF16_PEAK,
            "counts": "frac: matrix-core flops the kernel issues (an fp32 operand that goes in as three "
                      "bf16 terms counts three times); frac_useful_flops: 2 x (factor sizes) per element, "
                      "what the transform needs"}
    del keep, ops
    torch.cuda.empty_cache()
    if with_cpu_baseline:
        base = cpu_baseline_other(torch, workload, seed)
        if base is not None:
            out["cpu_baseline"] = base
    return out


API_FORMATS = (
    # format, weight scheme, algorithmic bytes per element and direction
    ("pack-quantized", dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=GROUP),
     2 + 2 / GROUP + 0.5),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="channel"), 3.0),
    ("nvfp4-pack-quantized", dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group",
                                  group_size=16), 2 + 1 / 16 + 0.5),
)


def api_level_format(torch, seed, steps, fmt, spec, bytes_per_element):
    """ModelCompressor.compress_model + decompress_model on a module tree of 224 bf16 Linear
    layers with the Llama-3-8B shapes (scales attached beforehand by the observer), one format"""
    from compressed_tensors_amd.compressors import ModelCompressor, apply_quantization_scheme
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme, observe_weight_qparams,
    )
    from compressed_tensors_amd.quantization.helpers import generate_gparam

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(seed)
    args = QuantizationArgs(**spec)

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            for name, r, c in LLAMA3_8B_LAYER:
                lin = torch.nn.Linear(c, r, bias=False, device="meta", dtype=torch.bfloat16)
                lin.to_empty(device=dev)
                lin.weight.data = (torch.randn(r, c, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
                lin.weight.requires_grad_(False)
                setattr(self, name, lin)

    model = torch.nn.Module()
    model.layers = torch.nn.ModuleList([Layer() for _ in range(32)])
    config = QuantizationConfig(
        config_groups={"group_0": QuantizationScheme(targets=["Linear"], weights=args)}, format=fmt)
    apply_quantization_scheme(model, config)
    n = 0
    for m in model.modules():
        if isinstance(m, torch.nn.Linear):
            if spec["strategy"] == "tensor_group":
                lo, hi = torch.aminmax(m.weight.data)
                gs = generate_gparam(lo.reshape(1), hi.reshape(1))
                m.register_parameter("weight_global_scale", torch.nn.Parameter(gs, requires_grad=False))
                scale, zp = observe_weight_qparams(m.weight.data, args, global_scale=gs)
            else:
                scale, zp = observe_weight_qparams(m.weight.data, args)
            m.register_parameter("weight_scale", torch.nn.Parameter(scale, requires_grad=False))
            m.register_parameter("weight_zero_point", torch.nn.Parameter(zp, requires_grad=False))
            n += m.weight.numel()
    mc = ModelCompressor(quantization_config=config)
    per_dir = bytes_per_element * n
    comp, deco = [], []
    for it in range(steps + 1):  # first pass is the warm-up
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        mc.compress_model(model)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        mc.decompress_model(model)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        if it:
            comp.append(t1 - t0)
            deco.append(t2 - t1)
    c_s, d_s = statistics.median(comp), statistics.median(deco)
    # the state-dict pathway: compress(model) -> compressed state dict, decompress(state dict, model)
    comp, deco = [], []
    for it in range(steps + 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        state = mc.compress(model)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        mc.decompress(state, model)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        del state
        if it:
            comp.append(t1 - t0)
            deco.append(t2 - t1)
    cs_s, ds_s = statistics.median(comp), statistics.median(deco)
    del model, mc
    torch.cuda.empty_cache()
    return {
        "compress_model_ms": c_s * 1e3, "decompress_model_ms": d_s * 1e3,
        "compress_GBs": per_dir / c_s / 1e9, "decompress_GBs": per_dir / d_s / 1e9,
        "roundtrip_GBs": 2 * per_dir / (c_s + d_s) / 1e9,
        "frac_of_hbm_peak": 2 * per_dir / (c_s + d_s) / 1e9 / HBM_PEAK_GBS,
        "state_dict_pathway": {
            "what": "compress(model) -> compressed state dict, decompress(state dict, model)",
            "compress_ms": cs_s * 1e3, "decompress_ms": ds_s * 1e3,
            "frac_of_hbm_peak": 2 * per_dir / (cs_s + ds_s) / 1e9 / HBM_PEAK_GBS},
        "passes": steps, "statistic": "median",
    }


def api_level_transform(torch, seed, steps):
    """TransformFactory.apply_to_model on the same module tree: a random-sign Hadamard rotation
    of block size 128 multiplied into the input side of all 224 weights (bf16 in, bf16 out:
    4 bytes per element), wall time incl. module matching and the parameter updates"""
    from compressed_tensors_amd.transform import TransformArgs, TransformFactory, TransformScheme

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(seed)

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            for name, r, c in LLAMA3_8B_LAYER:
                lin = torch.nn.Linear(1, 1, bias=False)
                lin.in_features, lin.out_features = c, r
                lin.weight.data = (torch.randn(r, c, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
                lin.weight.requires_grad_(False)
                setattr(self, name, lin)

    model = torch.nn.Module()
    model.layers = torch.nn.ModuleList([Layer() for _ in range(32)])
    n = sum(m.weight.numel() for m in model.modules() if isinstance(m, torch.nn.Linear))
    scheme = TransformScheme(type="random-hadamard", head_dim=128,
                             apply=[TransformArgs(targets="Linear", location="weight_input")])
    times = []
    for it in range(steps + 1):  # first pass is the warm-up
        factory = TransformFactory.from_scheme(scheme, name="R", seed=seed)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        factory.apply_to_model(model, use_tqdm=False)
        torch.cuda.synchronize()
        if it:
            times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    del model
    torch.cuda.empty_cache()
    return {"what": "TransformFactory.apply_to_model: random-hadamard, head_dim 128, weight_input of 224 "
                    "torch.nn.Linear (bf16, Llama-3-8B shapes)",
            "apply_to_model_ms": t * 1e3, "GBs": 4 * n / t / 1e9,
            "frac_of_hbm_peak": 4 * n / t / 1e9 / HBM_PEAK_GBS, "passes": steps, "statistic": "median"}


def api_level(torch, seed, steps):
    """the cost of the host mirror above the C ABI, next to the kernel-level figures: the
    headline's format at the top level of the result, the int8 / fp8 and nvfp4 formats under
    `other_formats`"""
    out = {"what": "ModelCompressor.compress_model + decompress_model, 224 torch.nn.Linear (bf16, on the "
                   "GPU) of the Llama-3-8B shapes, pack-quantized W4A16 g128, wall time incl. the Python "
                   "harness, parameter swaps and allocation of the outputs"}
    out.update(api_level_format(torch, seed, steps, *API_FORMATS[0]))
    out["other_formats"] = {fmt: api_level_format(torch, seed, steps, fmt, spec, bpe)
                            for fmt, spec, bpe in API_FORMATS[1:]}
    out["transform"] = api_level_transform(torch, seed, steps)
    return out


OTHER_WORKLOADS = ("fp8-w8a8", "sparse", "nvfp4", "hadamard", "one-shot", "standalone")

MAX_LINE = 1500  # characters of the line on stdout: what reads it keeps a short tail only


def _sig(x, digits=4):
    """floats to a few significant digits (the full figures are in the details file)"""
    if isinstance(x, float):
        return float(f"{x:.{digits}g}")
    return x


def short_line(out, details_path=None):
    """the one line that goes to stdout: the contract's fields, the roofline of the dominant
    kernel, the CPU baseline, and one number for each other configuration"""
    def pick(d, keys):
        return {k: _sig(d[k]) for k in keys if k in d}

    line = {k: _sig(out[k]) for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                      "higher_is_better", "scaling", "vs_baseline", "dtype", "data")
            if k in out}
    line["dtype"] = str(out.get("dtype", "")).split(" ")[0]
    line["config"] = pick(out.get("config", {}), ("workload", "tensors", "elements", "group_size", "seed"))
    line["roofline"] = pick(out["roofline"], ("bound", "kernel", "achieved", "peak", "unit", "frac",
                                              "traffic", "achieved_bytes_per_launch", "avg_launch_ms",
                                              "launches_per_step"))
    if "cpu_baseline" in out:
        base = pick(out["cpu_baseline"], ("value", "unit", "cores", "kind", "seconds"))
        base["sample"] = str(out["cpu_baseline"].get("sample_short") or out["cpu_baseline"].get("sample", ""))[:120]
        line["cpu_baseline"] = base
    if "parity" in out:
        line["parity"] = "bit-exact vs oracle (row slices, before timing)"
    if "configs" in out:
        # per configuration: algorithmic bytes of its operations / the sum of their GPU times, as a
        # fraction of the HBM peak, and the lowest fraction among them (comparison lines aside)
        def own(r):
            return [o for o in r["operations"] if not o["for_comparison_only"]]
        line["configs_frac"] = {
            w: [_sig(sum(o["algorithmic_bytes"] for o in own(r)) / sum(o["ms"] for o in own(r)) / 1e6 / HBM_PEAK_GBS, 3),
                _sig(min(o["frac_of_hbm_peak"] for o in own(r)), 3)]
            for w, r in out["configs"].items()}
        line["configs_frac_is"] = "[all operations, slowest operation]"
    if "mfma_utilisation" in out:
        line["mfma_frac"] = _sig(out["mfma_utilisation"]["frac"], 3)
    if "api_level" in out:
        line["api_level"] = pick(out["api_level"], ("frac_of_hbm_peak", "compress_model_ms", "decompress_model_ms"))
        if "state_dict_pathway" in out["api_level"]:
            line["api_level"]["state_dict_pathway"] = _sig(out["api_level"]["state_dict_pathway"]["frac_of_hbm_peak"], 3)
        for fmt, res in out["api_level"].get("other_formats", {}).items():
            line["api_level"][fmt] = _sig(res["frac_of_hbm_peak"], 3)
        if "transform" in out["api_level"]:
            line["api_level"]["hadamard128"] = _sig(out["api_level"]["transform"]["frac_of_hbm_peak"], 3)
    if details_path:
        line["details"] = os.path.relpath(details_path, ROOT)
    text = json.dumps(line, separators=(",", ":"))
    if len(text) > MAX_LINE:  # never happens with the fields above; drop the optional ones if it does
        for k in ("details", "parity", "configs_frac", "api_level", "mfma_frac"):
            line.pop(k, None)
            text = json.dumps(line, separators=(",", ":"))
            if len(text) <= MAX_LINE:
                break
    return text


def emit(out, details_path):
    """full result -> the details file (and stderr if the file cannot be written); short line -> stdout"""
    full = json.dumps(out, indent=1)
    written = None
    try:
        Path(details_path).parent.mkdir(parents=True, exist_ok=True)
        Path(details_path).write_text(full + "\n")
        written = details_path
    except OSError as e:
        print(f"bench.py: details not written ({e}); they follow on stderr", file=sys.stderr)
        print(full, file=sys.stderr)
    print(short_line(out, written), flush=True)


def headline(torch, a):
    from compressed_tensors_amd import _lib
    from compressed_tensors_amd.compressors.pack_quantized import PackedWeightBatch
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams

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

    # ---- parity spot check against the oracle (outside the timed region): the first, a
    # middle and the last rows of three tensors, the last tensor of the set among them
    from oracle import pack as opack
    from oracle import quant as oquant

    oargs = oquant._Args(num_bits=4, type="int", symmetric=True, strategy="group", group_size=GROUP)
    batch.compress()
    batch.decompress()
    torch.cuda.synchronize()
    checked = []
    for t in sorted({0, len(entries) // 2, len(entries) - 1}):
        n_rows = entries[t]["weight"].shape[0]
        for rows in (slice(0, 32), slice(n_rows // 2, n_rows // 2 + 32), slice(n_rows - 32, n_rows)):
            w0, s0, z0 = (entries[t][k][rows].cpu() for k in ("weight", "scale", "zero_point"))
            want = opack.pack_quantized_compress(w0, s0, oargs, zero_point=z0)
            assert torch.equal(batch.packed[t][rows].cpu(), want["weight_packed"]), "compress parity"
            want_d = opack.pack_quantized_decompress(dict(want, weight_scale=s0), oargs)
            assert torch.equal(batch.dense[t][rows].cpu().view(torch.int16), want_d.view(torch.int16)), \
                "decompress parity"
        checked.append(entries[t]["name"])

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
    traffic, traffic_source = measured_traffic(a.workload, dom)

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
        "dtype": "bf16 (every operation of the chain rounds to bf16, as the reference's does; codes are int4)",
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
            "traffic_source": traffic_source,
            "avg_launch_ms": dom_ms / n_launch,
            "launches_per_step": n_launch,
            "compress_GBs": comp_gbs,
            "decompress_GBs": deco_gbs,
            "compress_ms": comp_ms,
            "decompress_ms": deco_ms,
        },
        "parity": "bit-exact vs oracle on the first, middle and last 32 rows of " + ", ".join(checked)
                  + " (checked before timing)",
    }
    del batch, entries
    torch.cuda.empty_cache()
    if not a.no_cpu_baseline:
        sample = LLAMA3_8B_LAYER * 4  # four layers of 32 (about 10 s of CPU work); the others are identical work
        if a.workload == "w4a16-4096":
            sample = [("w", 4096, 4096)]
        out["cpu_baseline"] = cpu_baseline(torch, sample, a.seed)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=None)
    ap.add_argument("--only-headline", action="store_true",
                    help="the default workload without the short runs of the other configurations")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--calib-copies", type=int, default=0,
                    help="launch N plain 1 GiB copies first (byte-counter calibration when profiling)")
    ap.add_argument("--only-op", default=None,
                    help="with --workload: time only the operations whose name contains this text")
    ap.add_argument("--details", default=str(ROOT / "gpurun_out" / "bench_details.json"),
                    help="file the full result goes to (per-operation tables of every configuration); "
                         "stdout carries one short line")
    a = ap.parse_args()
    if a.gpus != 1:
        raise SystemExit(
            "bench.py measures one GPU: this path shards by whole tensors with no exchange "
            "step, and no multi-GPU figure is produced (run with --gpus 1)"
        )

    import torch

    from compressed_tensors_amd import _lib

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    _lib.load()
    everything = a.workload is None and not a.only_headline
    if a.workload is None:
        a.workload = "llama3-8b-w4a16"
    if a.workload == "api":
        print(json.dumps({k: _sig(v) for k, v in api_level(torch, a.seed, a.steps).items()}))
        return
    if a.workload in OTHER_WORKLOADS:
        emit(run_other(torch, a.workload, a.seed, a.steps, a.warmup, not a.no_cpu_baseline, a.only_op),
             a.details)
        return
    out = headline(torch, a)
    if everything:
        # the other configurations of the path, a few steps each
        steps, warmup = min(a.steps, 5), min(a.warmup, 2)
        out["configs"] = {}
        for w in OTHER_WORKLOADS:
            r = run_other(torch, w, a.seed, steps, warmup, not a.no_cpu_baseline)
            out["configs"][w] = {k: r[k] for k in ("metric", "value", "unit", "steps", "ms_per_step_gpu",
                                                   "roofline", "mfma_utilisation", "operations",
                                                   "cpu_baseline") if k in r}
        out["api_level"] = api_level(torch, a.seed, min(a.steps, 5))
    emit(out, a.details)


if __name__ == "__main__":
    main()
