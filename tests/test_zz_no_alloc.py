"""The allocation-free variant of bitmask decompress (scratch in a device array inside
the library) gives the bits of the entry point that takes a caller's scratch buffer."""
import pytest
import torch

from gpu_util import announce
from oracle import sparse as osp


def _case(rows, cols, dtype, sparsity, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, cols, generator=g) * 0.02).to(dtype)
    x[torch.rand(rows, cols, generator=g) < sparsity] = 0
    return x


def _run_both(ctmi, _lib, x, gpu):
    """-> (output of ctmi_bitmask_decompress with a caller's scratch, output of the static
    variant, the oracle's dense tensor); every buffer is allocated before either call"""
    rows, cols = x.shape
    values, bitmask, _ = osp.bitmask_compress(x)
    want = osp.bitmask_decompress(values, bitmask, [rows, cols])
    d_values, d_bitmask = values.to(gpu), bitmask.to(gpu).contiguous()
    tmp = torch.empty(ctmi.ctmi_bitmask_tmp_bytes(rows, cols), dtype=torch.uint8, device=gpu)
    # poison the outputs: every element must be written by the call
    out_a = torch.full((rows, cols), 7.0, dtype=x.dtype, device=gpu)
    out_b = torch.full((rows, cols), 9.0, dtype=x.dtype, device=gpu)
    stream = _lib.stream_of(gpu)
    before = torch.cuda.memory_allocated(gpu)
    _lib.check(ctmi.ctmi_bitmask_decompress(d_values.data_ptr(), d_values.numel(), x.element_size(),
                                            d_bitmask.data_ptr(), None, out_a.data_ptr(),
                                            tmp.data_ptr(), rows, cols, stream))
    _lib.check(ctmi.ctmi_bitmask_decompress_static(d_values.data_ptr(), d_values.numel(),
                                                   x.element_size(), d_bitmask.data_ptr(),
                                                   out_b.data_ptr(), rows, cols, stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(gpu) == before
    return out_a.cpu(), out_b.cpu(), want


def _bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


@pytest.mark.gpu
def test_static_scratch_decompress_matches_the_scratch_argument_one(ctmi, gpu):
    from compressed_tensors_amd import _lib

    # two calls in a row on one stream, the second smaller: what the first left in the
    # shared scratch must not leak into the second.  Then the other kernel families
    # behind the entry point (row kernels for ragged shapes, 4-byte elements).
    cases = [(2048, 8192, torch.bfloat16, 0.5, 1), (96, 4096, torch.bfloat16, 0.7, 2),
             (33, 2050, torch.bfloat16, 0.5, 3), (5, 1040, torch.float32, 0.8, 4),
             (64, 4096, torch.float16, 0.0, 5)]
    for rows, cols, dtype, sparsity, seed in cases:
        announce("static-scratch decompress", rows, cols, dtype, sparsity)
        x = _case(rows, cols, dtype, sparsity, seed)
        a, b, want = _run_both(ctmi, _lib, x, gpu)
        assert torch.equal(_bits(a), _bits(want)), "scratch-argument entry point vs oracle"
        assert torch.equal(_bits(b), _bits(a)), "static-scratch entry point vs scratch-argument one"


@pytest.mark.gpu
def test_static_scratch_decompress_replays_from_a_captured_graph(ctmi, gpu):
    """the caller the entry point is for: captured once into a HIP graph (nothing is allocated
    and nothing cleared by a memset node), replayed several times with new inputs copied into
    the same buffers and eager work in between; every replay equals the eager call"""
    from compressed_tensors_amd import _lib

    announce("static-scratch decompress in a captured graph")
    rows, cols = 1024, 4096
    packed = []
    for seed, sparsity in ((11, 0.5), (12, 0.9), (13, 0.2), (14, 0.5)):
        values, bitmask, _ = osp.bitmask_compress(_case(rows, cols, torch.bfloat16, sparsity, seed))
        packed.append((values.to(gpu), bitmask.to(gpu).contiguous()))
    room = max(v.numel() for v, _ in packed)
    d_values = torch.zeros(room, dtype=torch.bfloat16, device=gpu)
    d_bitmask = torch.zeros_like(packed[0][1])
    out = torch.empty((rows, cols), dtype=torch.bfloat16, device=gpu)
    tmp = torch.empty(ctmi.ctmi_bitmask_tmp_bytes(rows, cols), dtype=torch.uint8, device=gpu)

    def load(k):
        d_values.zero_()
        d_values[: packed[k][0].numel()].copy_(packed[k][0])
        d_bitmask.copy_(packed[k][1])

    def call():
        # nvalues is fixed in the captured call: the buffer's size; what lies behind a
        # tensor's own values is zero and is never reached by a set bit
        _lib.check(ctmi.ctmi_bitmask_decompress_static(d_values.data_ptr(), room, 2, d_bitmask.data_ptr(),
                                                       out.data_ptr(), rows, cols, _lib.stream_of(gpu)))

    load(0)
    call()  # the per-device set-up of the entry point happens outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for k in (1, 2, 3, 0, 2):
        load(k)
        want = torch.empty_like(out)
        _lib.check(ctmi.ctmi_bitmask_decompress(d_values.data_ptr(), room, 2, d_bitmask.data_ptr(), None,
                                                want.data_ptr(), tmp.data_ptr(), rows, cols,
                                                _lib.stream_of(gpu)))
        out.fill_(3.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(out.cpu()), _bits(want.cpu())), f"replay with tensor {k}"


def test_static_scratch_rejects_what_does_not_fit(ctmi):
    """refused on the host, before any HIP call: runs without a GPU"""
    from compressed_tensors_amd import _lib

    limit = ctmi.ctmi_bitmask_decompress_static_max_bytes()
    assert limit == 4 << 20
    rows, cols = 1 << 18, 4096  # 16 bytes a row alone exceed the buffer
    assert ctmi.ctmi_bitmask_tmp_bytes(rows, cols) > limit
    rc = ctmi.ctmi_bitmask_decompress_static(0x1000, 16, 2, 0x2000, 0x3000, rows, cols, None)
    assert rc == _lib.CTMI_ERR_VALUE
    assert "static buffer" in ctmi.ctmi_last_error().decode()
