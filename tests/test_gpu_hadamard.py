"""GPU parity: Hadamard transform apply vs the oracle (fp64 / fp32 matmul by the
explicit matrix): within one ulp of the output dtype."""
import pytest
import torch

from gpu_util import announce, assert_bit_equal
from oracle import hadamard as oh

pytestmark = pytest.mark.gpu


# elements (of all 16-bit comparisons of this file) that were more than one ulp off and passed
# on the fp32-accumulation allowance; printed by the last test
ALLOWANCE = {"elements": 0, "leaning": 0}
ALLOWANCE_FRACTION = 1e-3


def _ulp(t: torch.Tensor) -> torch.Tensor:
    """spacing of t's dtype at |t| (as float64)"""
    bits = {torch.bfloat16: 8, torch.float16: 11, torch.float32: 24}[t.dtype]
    mag = t.double().abs().clamp_min(2.0 ** (-14 if t.dtype == torch.float16 else -126))
    return torch.exp2(torch.floor(torch.log2(mag)) - (bits - 1))


def _assert_within_ulp(got, exact, what, ulps=1.0):
    got = got.cpu()
    assert got.dtype == exact.dtype and got.shape == exact.shape, what
    err = (got.double() - exact.double()).abs()
    if exact.dtype == torch.float32:
        # fp32 accumulation of n terms: rtol 1e-5 of the value plus the same fraction of the
        # largest term scale of the row (cancellation makes a pure per-value bound meaningless)
        tol = 1e-5 * exact.double().abs() + 1e-5 * exact.double().abs().amax(-1, keepdim=True)
    else:
        # one ulp of the output dtype, plus the fp32 accumulation error of the n-term sums
        # (2^-21 of the row's scale): it only shows where cancellation leaves an output
        # thousands of times smaller than its terms, e.g. in float16's subnormal range
        tol = ulps * _ulp(exact) + 2.0 ** -21 * exact.double().abs().amax(-1, keepdim=True)
        # how many elements lean on that second term: outputs next to a rounding boundary or far
        # below the row's scale.  It stays a small fraction (ALLOWANCE_FRACTION) of the tensor.
        leaning = int((err > ulps * _ulp(exact)).sum())
        ALLOWANCE["elements"] += err.numel()
        ALLOWANCE["leaning"] += leaning
        assert leaning <= max(2, ALLOWANCE_FRACTION * err.numel()), \
            f"{what}: {leaning} of {err.numel()} elements are more than {ulps} ulp off (within the accumulation allowance)"
    bad = err > tol
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} elements off by more than {ulps} ulp; max ratio {(err / tol).max():.2f}"


def _reference(weight64, value, location, inverse=False, module_type=torch.nn.Linear, perm=None):
    """fp64 application rounded once to value.dtype: the exact answer"""
    return oh.hadamard_forward(weight64, value, location, module_type, inverse, perm)


SIZES = [32, 64, 128, 1024, 2048, 4096, 8192]


@pytest.mark.parametrize("kernel", ["mfma", "butterfly"])
@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_sylvester_apply(n, dtype, kernel, gpu):
    """both implementations of x -> x H_n: products with the factors of H_n on the matrix
    cores, and (n >= 1024) butterflies in registers"""
    from compressed_tensors_amd import _lib
    from compressed_tensors_amd.transform import hadamard_apply, hadamard_factors

    announce("hadamard_apply", n, dtype, kernel)
    a, b = hadamard_factors(n)
    if kernel == "mfma" and not _lib.load().ctmi_hadamard_supported(a, b, _lib.dtype_code(dtype)):
        pytest.skip("factorisation not built for this dtype")
    if kernel == "butterfly" and not _lib.load().ctmi_sylvester_supported(n, _lib.dtype_code(dtype)):
        with pytest.raises(NotImplementedError):
            hadamard_apply(torch.zeros(1, n, dtype=dtype, device=gpu), n, kernel=kernel)
        return
    g = torch.Generator().manual_seed(n)
    rows = 37 if n <= 2048 else 9
    x = torch.randn(rows, 2 * n if n <= 1024 else n, generator=g).to(dtype)
    q = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).double()
    h = oh.deterministic_hadamard_matrix(n, torch.float64)
    y = hadamard_apply(x.to(gpu), n, kernel=kernel)
    _assert_within_ulp(y, _reference(h, x, "input"), "plain")
    y = hadamard_apply(x.to(gpu), n, sign_in=q.float(), kernel=kernel)
    _assert_within_ulp(y, _reference(q.unsqueeze(1) * h, x, "input"), "sign_in")
    y = hadamard_apply(x.to(gpu), n, sign_out=q.float(), kernel=kernel)
    _assert_within_ulp(y, _reference((q.unsqueeze(1) * h).T, x, "input"), "sign_out")
    y = hadamard_apply(x.to(gpu), n, sign_in=q.float(), sign_out=q.flip(0).float(), kernel=kernel)
    _assert_within_ulp(y, _reference(q.unsqueeze(1) * h * q.flip(0), x, "input"), "both signs")


def test_butterfly_kernel_runs_of_many_rows(gpu):
    """more runs than workgroups are resident (every workgroup takes several, with the next
    run's loads and first pass under way), for each size: every row against the fp64 product"""
    from compressed_tensors_amd.transform import hadamard_apply

    for n, rows in ((1024, 40_000), (2048, 20_000), (4096, 5_000), (8192, 4_099)):
        announce("butterfly rows", n, rows)
        g = torch.Generator(device=gpu).manual_seed(n)
        x = torch.randn(rows, n, generator=g, device=gpu).bfloat16()
        y = hadamard_apply(x, n, kernel="butterfly")
        h = oh.deterministic_hadamard_matrix(n, torch.float64).to(gpu)
        for r0 in range(0, rows, 4096):
            want = (x[r0:r0 + 4096].double() @ h / n ** 0.5).bfloat16()
            _assert_within_ulp(y[r0:r0 + 4096], want.cpu(), f"n={n} rows {r0}..")


def test_explicit_small_matrix(gpu):
    from compressed_tensors_amd.transform import hadamard_apply

    announce("explicit matrix 64")
    g = torch.Generator().manual_seed(3)
    m = (torch.randint(0, 2, (64, 64), generator=g) * 2 - 1).double()  # any +-1 matrix
    x = torch.randn(50, 192, generator=g).bfloat16()
    y = hadamard_apply(x.to(gpu), 64, matrix_t=m.T.contiguous())
    _assert_within_ulp(y, _reference(m, x, "input"), "explicit")


LOCS = [("input", False), ("input", True), ("weight_input", False), ("weight_input", True),
        ("weight_output", False), ("weight_output", True), ("output", False)]


@pytest.mark.parametrize("kind", ["hadamard", "random-hadamard"])
@pytest.mark.parametrize("location,inverse", LOCS)
def test_transform_objects(kind, location, inverse, gpu):
    from compressed_tensors_amd.transform import (
        TransformArgs, TransformFactory, TransformScheme,
    )

    announce("transform", kind, location, inverse)
    scheme = TransformScheme(type=kind, apply=[], head_dim=None)
    factory = TransformFactory.from_scheme(scheme, name="t", seed=11)
    linear = torch.nn.Linear(256 if location != "weight_output" else 128, 128, bias=False)
    if location in ("weight_output", "output"):
        linear = torch.nn.Linear(64, 128, bias=False)
    else:
        linear = torch.nn.Linear(128, 64, bias=False)
    args = TransformArgs(targets=["Linear"], location=location, inverse=inverse)
    tfm = factory.create_transform(linear, args)
    weight64 = tfm.weight.double()
    g = torch.Generator().manual_seed(5)
    if location in ("weight_input", "weight_output"):
        value = (torch.randn(linear.out_features, linear.in_features, generator=g) * 0.02).bfloat16()
    elif location == "input":
        value = torch.randn(3, 7, 128, generator=g).bfloat16()
    else:
        value = torch.randn(3, 7, 128, generator=g).bfloat16()
    got = tfm(value.to(gpu))
    want = _reference(weight64, value, location, inverse)
    _assert_within_ulp(got, want, f"{kind} {location} inverse={inverse}")


def test_multihead_and_permutation(gpu):
    from compressed_tensors_amd.transform import (
        TransformArgs, TransformFactory, TransformScheme,
    )

    announce("transform head_dim + randomize")
    scheme = TransformScheme(type="random-hadamard", head_dim=64, randomize=True)
    factory = TransformFactory.from_scheme(scheme, name="t", seed=3)
    linear = torch.nn.Linear(256, 128, bias=False)
    g = torch.Generator().manual_seed(6)
    for location, value in (("input", torch.randn(4, 9, 256, generator=g).bfloat16()),
                            ("weight_input", (torch.randn(128, 256, generator=g) * 0.02).bfloat16())):
        tfm = factory.create_transform(linear, TransformArgs(["Linear"], location))
        assert tfm.size == 64 and tfm.perm is not None
        want = _reference(tfm.weight.double(), value, location, perm=tfm.perm)
        _assert_within_ulp(tfm(value.to(gpu)), want, f"multihead {location}")


def test_transform_algebra_on_gpu(gpu):
    """output_tfm(input_tfm(x) @ (U W V)^T) == x W^T at atol 1e-5 in fp32"""
    from compressed_tensors_amd.transform import (
        TransformArgs, TransformFactory, TransformScheme,
    )

    announce("transform algebra")
    scheme = TransformScheme(type="random-hadamard")
    fac = TransformFactory.from_scheme(scheme, name="t", seed=0)
    lin = torch.nn.Linear(128, 64, bias=False)
    g = torch.Generator().manual_seed(9)
    w = torch.randn(64, 128, generator=g).to(gpu)
    x = torch.randn(5, 128, generator=g).to(gpu)
    t_in = fac.create_transform(lin, TransformArgs(["Linear"], "input"))
    t_wi = fac.create_transform(lin, TransformArgs(["Linear"], "weight_input", inverse=True))
    t_wo = fac.create_transform(lin, TransformArgs(["Linear"], "weight_output"))
    t_out = fac.create_transform(lin, TransformArgs(["Linear"], "output", inverse=True))
    y = t_out(t_in(x) @ t_wo(t_wi(w)).T)
    assert torch.allclose(y, x @ w.T, atol=1e-4)


def test_large_activation_properties(gpu):
    """full-size: 8192 x 4096 bf16 activations, block 128 and full 4096: sampled
    rows against fp64, and an involution check (H H^T / n = I) on the whole tensor"""
    from compressed_tensors_amd.transform import hadamard_apply

    announce("hadamard large")
    g = torch.Generator().manual_seed(0)
    x = torch.randn(8192, 4096, generator=g).bfloat16()
    xg = x.to(gpu)
    for n in (128, 4096):
        q = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
        y = hadamard_apply(xg, n, sign_in=q)
        rows = torch.tensor([0, 1, 4095, 8191])
        w = q.double().unsqueeze(1) * oh.deterministic_hadamard_matrix(n, torch.float64)
        _assert_within_ulp(y[rows.to(gpu)], _reference(w, x[rows], "input"), f"rows n={n}")
        back = hadamard_apply(y, n, sign_out=q)  # times W^T / sqrt(n): undoes it up to bf16 rounding
        rel = (back.float() - xg.float()).abs().max() / xg.float().abs().max()
        assert float(rel) < 2e-2


@pytest.mark.parametrize("n,shape,kernel", [
    (128, (64, 512), None), (128, (37, 256), None), (64, (33, 192), None), (32, (19, 96), None),
    (4096, (37, 4096), "mfma"), (4096, (5, 8192), "mfma"), (2048, (21, 4096), "mfma"),
    (4096, (37, 4096), "butterfly"), (4096, (2100, 8192), "butterfly"), (2048, (21, 4096), "butterfly"),
    (1024, (300, 3072), "butterfly"), (8192, (11, 8192), "butterfly"), (8192, (3000, 8192), None)])
def test_fused_rotation_quantization_packing(n, shape, kernel, gpu):
    """ctmi_hadamard_quant_pack == hadamard_apply -> min-max observer -> pack-quantized
    compress, bit for bit (each of which is checked against the oracle on its own), and
    the whole chain against the oracle's."""
    from oracle import pack as op
    from oracle import quant as oq
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams
    from compressed_tensors_amd.transform import hadamard_apply, hadamard_quantize_pack

    announce("fused hadamard + int4 + pack", n, shape, kernel)
    kern = dict(kernel=kernel) if n > 128 else {}
    g = torch.Generator().manual_seed(3 * n + shape[0])
    x = (torch.randn(shape, generator=g) * 0.02).bfloat16()
    group = min(n, 128)  # transforms of 2048 / 4096 elements feed groups of 128
    if n <= 128:
        x[0, :n] = 0  # an all-zero group: scale clamps to eps
    else:
        x[1] = 0      # a rotated row of zeros: every group of it
    q = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    args = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group", group_size=group)
    for signs in (dict(), dict(sign_in=q), dict(sign_out=q)):
        fused = hadamard_quantize_pack(x.to(gpu), n, args, return_rotated=True, **signs, **kern)
        y = hadamard_apply(x.to(gpu), n, **signs, **kern)
        no_copy = hadamard_quantize_pack(x.to(gpu), n, args, **signs, **kern)
        assert torch.equal(no_copy["weight_packed"], fused["weight_packed"]) and "rotated" not in no_copy
        # (bit for bit up to the sign of an exact zero: kernels that apply an output sign to the
        # rounded result give -0 where kernels that fold it into the matrix give +0)
        unsigned_zero = lambda t: torch.where(t == 0, torch.zeros_like(t), t).view(torch.int16)
        assert torch.equal(unsigned_zero(fused["rotated"]), unsigned_zero(y)), "rotated tensor"
        scale, zp = observe_weight_qparams(y, args)
        comp = BaseCompressor.load_from_registry("pack-quantized")
        want = comp.compress_weight(weight=y, scale=scale, quantization_args=args, zero_point=zp)
        assert torch.equal(fused["weight_scale"].view(torch.int16), scale.view(torch.int16)), "scales"
        assert torch.equal(fused["weight_packed"], want["weight_packed"]), "packed codes"
        assert fused["weight_shape"].tolist() == list(shape)
        # the oracle's chain on the same rotated tensor
        oargs = oq._Args(num_bits=4, type="int", symmetric=True, strategy="group", group_size=group)
        yc = y.cpu()
        o_scale, o_zp = oq.observe_weight(yc, oargs)
        o_packed = op.pack_quantized_compress(yc, o_scale, oargs, zero_point=o_zp)["weight_packed"]
        assert torch.equal(fused["weight_scale"].cpu().view(torch.int16), o_scale.view(torch.int16))
        assert torch.equal(fused["weight_packed"].cpu(), o_packed)


@pytest.mark.parametrize("n,dtype", [(128, torch.bfloat16), (64, torch.float16), (32, torch.bfloat16),
                                     (4096, torch.bfloat16), (1024, torch.float16), (2048, torch.bfloat16),
                                     (128, torch.float32), (8192, torch.float16), (4096, torch.float32)])
def test_many_tensors_in_one_call(n, dtype, gpu):
    """hadamard_apply_many == hadamard_apply tensor by tensor, bit for bit: more tensors than
    one launch takes (8), sizes that differ, a tensor that ends in a ragged group of
    sub-rows (it gets a call of its own), an empty one; fp32 goes tensor by tensor"""
    from compressed_tensors_amd.transform import hadamard_apply, hadamard_apply_many

    announce("hadamard many", n, dtype)
    g = torch.Generator().manual_seed(n)
    q_in = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    q_out = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    rows = [16, 48, 5, 64, 1, 32, 16, 80, 16, 33, 0]
    xs = [(torch.randn(r, 2 * n if n <= 128 else n, generator=g) * 0.05).to(dtype).to(gpu) for r in rows]
    for signs in (dict(), dict(sign_in=q_in, sign_out=q_out)):
        got = hadamard_apply_many(xs, n, **signs)
        assert len(got) == len(xs)
        for i, (x, y) in enumerate(zip(xs, got)):
            assert y.shape == x.shape
            if x.numel():
                assert_bit_equal(y, hadamard_apply(x, n, **signs), f"tensor {i} ({rows[i]} rows)")


@pytest.mark.parametrize("signs", ["none", "in", "out", "both"])
def test_sylvester128_without_a_matrix(signs, gpu):
    """Sylvester's matrix of 128 on bfloat16 tensors runs from a kernel that keeps no matrix in
    memory (no matrix_t): the same bits as the kernel that is handed the matrix, one tensor
    per call and several per call, whole and ragged groups of 16 sub-rows, in place; and the
    fp64 product by the explicit matrix within one ulp"""
    from compressed_tensors_amd import _lib
    from compressed_tensors_amd.transform import hadamard_apply, hadamard_apply_many
    from compressed_tensors_amd.transform.hadamard import _sylvester_bf16

    announce("sylvester 128, no matrix", signs)
    n = 128
    g = torch.Generator().manual_seed(5)
    q_in = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float() if signs in ("in", "both") else None
    q_out = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float() if signs in ("out", "both") else None
    kw = dict(sign_in=q_in, sign_out=q_out)
    shapes = [(16, 128), (64, 512), (5, 256), (33, 384), (1, 128), (2048, 256), (7, 1152), (48, 128), (16, 256), (3, 128)]
    xs = [(torch.randn(s, generator=g) * 0.05).bfloat16().to(gpu) for s in shapes]
    xs[2][0, 3] = float("inf")
    xs[3][1, 200] = float("nan")
    matrix_t = _sylvester_bf16(n, gpu)
    lib = _lib.load()
    many = hadamard_apply_many(xs, n, **kw)
    with_matrix = hadamard_apply_many(xs, n, matrix_t=matrix_t, **kw)
    h = oh.deterministic_hadamard_matrix(n, dtype=torch.float64)
    def same(got, want, what):  # bit for bit; a NaN is a NaN whatever its sign bit
        got, want = got.cpu(), want.cpu()
        nan = torch.isnan(want.float())
        assert torch.equal(torch.isnan(got.float()), nan), f"{what}: NaNs"
        assert_bit_equal(torch.where(nan, torch.zeros_like(got), got), torch.where(nan, torch.zeros_like(want), want), what)

    for i, (x, y, w) in enumerate(zip(xs, many, with_matrix)):
        same(y, w, f"tensor {i} {tuple(x.shape)}: no matrix vs matrix")
        same(hadamard_apply(x, n, **kw), w, f"tensor {i}: single call")
        if i not in (2, 3):
            v = x.cpu().double().reshape(-1, n)
            if q_in is not None:
                v = v * q_in.double()
            exact = v @ h
            if q_out is not None:
                exact = exact * q_out.double()
            exact = (exact / n ** 0.5).reshape(x.shape).to(torch.bfloat16)
            _assert_within_ulp(y, exact, f"tensor {i} vs fp64")
    # in place
    z = xs[1].clone()
    lib_jobs = (_lib.HadamardJob * 1)()
    lib_jobs[0].x, lib_jobs[0].out, lib_jobs[0].numel = z.data_ptr(), z.data_ptr(), z.numel()
    s_in = None if q_in is None else q_in.to(gpu)
    s_out = None if q_out is None else q_out.to(gpu)
    _lib.check(lib.ctmi_hadamard_apply_many(lib_jobs, 1, _lib.dtype_code(z.dtype), 1, n, None, None,
                                            _lib.ptr(s_in), _lib.ptr(s_out), _lib.stream_of(z.device)))
    assert_bit_equal(z, with_matrix[1].cpu(), "in place")


@pytest.mark.parametrize("n", [128, 4096, 2048, 1024])
def test_fused_many_tensors_in_one_call(n, gpu):
    """hadamard_quantize_pack_many == hadamard_quantize_pack tensor by tensor"""
    from compressed_tensors_amd.quantization import QuantizationArgs
    from compressed_tensors_amd.transform import hadamard_quantize_pack, hadamard_quantize_pack_many

    announce("fused hadamard many", n)
    g = torch.Generator().manual_seed(77)
    q = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    args = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    shapes = [(64, 512), (37, 256), (16, 128), (5, 1024), (128, 256), (1, 128), (48, 384), (33, 128), (96, 640),
              (7, 256)]
    if n > 128:
        shapes = [(r, n * (1 + i % 2)) for i, (r, _) in enumerate(shapes)]
    xs = [(torch.randn(s, generator=g) * 0.02).bfloat16().to(gpu) for s in shapes]
    for signs in (dict(), dict(sign_in=q)):
        got = hadamard_quantize_pack_many(xs, n, args, **signs)
        for i, (x, out) in enumerate(zip(xs, got)):
            want = hadamard_quantize_pack(x, n, args, **signs)
            assert_bit_equal(out["weight_packed"], want["weight_packed"], f"packed {i}")
            assert_bit_equal(out["weight_scale"], want["weight_scale"], f"scale {i}")
            assert out["weight_shape"].tolist() == list(shapes[i])


# ---------------------------------------------------------------- explicit factors (ctmi_kron_matmul)


def _sylvester64(n):
    return oh.deterministic_hadamard_matrix(n, torch.float64)


@pytest.mark.parametrize("h,b", [(12, 2), (12, 64), (20, 8), (28, 128), (224, 64), (1, 256), (4, 64),
                                 (8, 64), (1, 8), (3, 1), (148, 128), (1, 512), (1, 2), (1, 16),
                                 (1, 1)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_kron_matmul(h, b, dtype, gpu):
    """x * diag(s_in) * (w (x) Sylvester(b)) * diag(s_out) / sqrt(h b) against fp64, for
    factors w that are not Hadamard matrices either; the run count is odd, so the last
    workgroup of the several-runs-per-workgroup layout is partly empty"""
    from compressed_tensors_amd.transform import kron_apply

    announce("kron_matmul", h, b, dtype)
    n = h * b
    g = torch.Generator().manual_seed(1000 * h + b)
    runs = 37 if n <= 4096 else 5
    x = torch.randn(runs, n, generator=g).to(dtype)
    w = torch.randn(h, h, generator=g).float() if h != 224 else (
        torch.randint(0, 2, (h, h), generator=g) * 2 - 1).float()
    s_in = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    s_out = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    dense = torch.kron(w.double(), _sylvester64(b))
    y = kron_apply(x.to(gpu), w, inner=b, sylvester=True)
    _assert_within_ulp(y, (x.double() @ dense / n ** 0.5).to(dtype), "plain")
    y = kron_apply(x.to(gpu), w, inner=b, sign_in=s_in, sign_out=s_out, sylvester=True)
    want = ((x.double() * s_in.double()) @ dense * s_out.double() / n ** 0.5).to(dtype)
    _assert_within_ulp(y, want, "signs")
    if b > 256:
        return
    # without the Sylvester factor: w (x) I, unscaled
    y = kron_apply(x.to(gpu), w, inner=b, sylvester=False)
    want = (x.double() @ torch.kron(w.double(), torch.eye(b, dtype=torch.float64))).to(dtype)
    _assert_within_ulp(y, want, "identity inner factor")


@pytest.mark.parametrize("h", [1, 3, 16, 100, 128, 313])
def test_block_matmul_entry_point(h, ctmi, gpu):
    """ctmi_block_matmul straight through the C ABI: every run of h values times an
    arbitrary matrix / sqrt(h); 70 runs = one full tile of 64 and a ragged one"""
    from compressed_tensors_amd import _lib

    announce("ctmi_block_matmul", h)
    g = torch.Generator().manual_seed(h)
    x = torch.randn(70, h, generator=g).bfloat16()
    w = torch.randn(h, h, generator=g)
    xg, wg = x.to(gpu), w.to(gpu)
    out = torch.empty_like(xg)
    _lib.check(ctmi.ctmi_block_matmul(xg.data_ptr(), out.data_ptr(), _lib.dtype_code(x.dtype),
                                      x.numel(), h, wg.data_ptr(), _lib.stream_of(gpu)))
    torch.cuda.synchronize()
    _assert_within_ulp(out, (x.double() @ w.double() / h ** 0.5).bfloat16(), f"h={h}")


def test_kron_matmul_refuses_what_does_not_fit(ctmi, gpu):
    from compressed_tensors_amd import _lib

    code = _lib.dtype_code(torch.bfloat16)
    assert ctmi.ctmi_kron_matmul_supported(224, 64, code) == 1
    assert ctmi.ctmi_kron_matmul_supported(313, 1, code) == 1
    assert ctmi.ctmi_kron_matmul_supported(314, 1, code) == 0
    assert ctmi.ctmi_kron_matmul_supported(12, 3, code) == 0      # inner size not a power of two
    assert ctmi.ctmi_kron_matmul_supported(12, 512, code) == 0    # more than 256 lanes
    assert ctmi.ctmi_kron_matmul_supported(1, 512, code) == 1     # plain Sylvester: in registers
    assert ctmi.ctmi_kron_matmul_supported(1, 1024, code) == 1    # ... and up to 8192 with the run in LDS
    assert ctmi.ctmi_kron_matmul_supported(1, 16384, code) == 0
    assert ctmi.ctmi_kron_matmul_supported(2, 1024, code) == 0
    assert ctmi.ctmi_kron_matmul_supported(256, 256, code) == 0   # 256 KB of LDS
    x = torch.zeros(314 * 4, dtype=torch.bfloat16, device=gpu)
    w = torch.zeros(314, 314, device=gpu)
    rc = ctmi.ctmi_block_matmul(x.data_ptr(), x.data_ptr(), code, x.numel(), 314, w.data_ptr(), None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED
    rc = ctmi.ctmi_kron_matmul(x.data_ptr(), x.data_ptr(), code, 100, 12, 2, w.data_ptr(), None, None,
                               1, 1.0, None)
    assert rc == _lib.CTMI_ERR_VALUE  # 100 is not a multiple of 24
    rc = ctmi.ctmi_kron_matmul(x.data_ptr(), x.data_ptr(), code, 1024, 1, 512, w.data_ptr(), None,
                               None, 0, 1.0, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED  # 512 lanes only for the Sylvester factor


@pytest.mark.parametrize("size", [768, 1600, 3584, 7168, 14336, 3072, 5120, 3840, 15360, 16384, 32, 256, 512, 16])
@pytest.mark.parametrize("location,inverse", [("input", False), ("weight_input", True),
                                              ("weight_output", False), ("output", True)])
def test_random_hadamard_of_any_table_size(size, location, inverse, gpu, hadamard_table_path,
                                           monkeypatch):
    """sizes K * 2^m from the table of known matrices (3584 = 28 * 128, 7168 = 224 * 32,
    14336 = 224 * 64: Llama-3's intermediate size; 3072 = 192 * 16, 5120 = 160 * 32, 3840 = 240 * 16
    and 15360 = 240 * 64 with this table), 16384 = Sylvester(128) as the block of 128 * 128, 32 (whose table entry is not Sylvester's) and the powers of two
    that have no matrix-core kernel: forward against the dense fp64 matrix the oracle
    builds with the reference's butterfly stages"""
    from compressed_tensors_amd.transform import (
        TransformArgs, TransformFactory, TransformScheme, load_hadamard_table,
    )
    from compressed_tensors_amd.transform import hadamard as product

    if size >= 768:  # these have a matrix-core kernel: the dense matrix must not be what ran
        def refuse(*a, **k):
            raise AssertionError(f"size {size} went through the dense matrix")
        monkeypatch.setattr(product, "apply_transform_weight", refuse)

    announce("random hadamard", size, location, inverse)
    scheme = TransformScheme(type="random-hadamard")
    factory = TransformFactory.from_scheme(scheme, name="t", seed=size, table_path=hadamard_table_path)
    other = 48
    if location in ("input", "weight_input"):
        linear = torch.nn.Linear(size, other, bias=False, device="meta")
    else:
        linear = torch.nn.Linear(other, size, bias=False, device="meta")
    tfm = factory.create_transform(linear, TransformArgs(["Linear"], location, inverse=inverse))
    assert tfm.size == size
    table = {k: v for k, v in load_hadamard_table(hadamard_table_path).items()}
    gen = torch.Generator().manual_seed(size)
    weight64 = oh.random_hadamard_matrix(size, dtype=torch.float64, gen=gen, table=table)
    g = torch.Generator().manual_seed(5)
    if location in ("weight_input", "weight_output"):
        value = (torch.randn(linear.out_features, linear.in_features, generator=g) * 0.02).bfloat16()
    else:
        value = torch.randn(3, 5, size, generator=g).bfloat16()
    got = tfm(value.to(gpu))
    _assert_within_ulp(got, _reference(weight64, value, location, inverse), f"{size} {location}")
    if size == 768:
        assert torch.equal(tfm.weight.double(), weight64)


@pytest.mark.parametrize("location", ["input", "weight_input", "weight_output", "output"])
@pytest.mark.parametrize("module_type", [torch.nn.Linear, torch.nn.Embedding])
def test_apply_transform_weight_runs_the_kernel(location, module_type, gpu, monkeypatch):
    """explicit 128 x 128 blocks (a head dimension) on a 512-wide value: every location
    and module kind against the oracle in fp64; torch.matmul must not be what ran"""
    from compressed_tensors_amd.transform import apply_transform_weight
    from compressed_tensors_amd.transform import hadamard as product

    announce("apply_transform_weight", location, module_type.__name__)
    if module_type is torch.nn.Embedding and location in ("input", "output"):
        pytest.skip("online locations do not depend on the module kind")
    g = torch.Generator().manual_seed(17)
    w = torch.randn(128, 128, generator=g).bfloat16()
    left = (module_type is torch.nn.Linear and location == "weight_output") or (
        module_type is torch.nn.Embedding and location == "weight_input")
    value = (torch.randn(512, 96, generator=g) if left else torch.randn(96, 512, generator=g)).bfloat16()
    calls = []
    real = product.kron_apply
    monkeypatch.setattr(product, "kron_apply", lambda *a, **k: calls.append(1) or real(*a, **k))
    got = apply_transform_weight(w.to(gpu), value.to(gpu), location, module_type)
    assert calls, "the HIP kernel was not used"
    want = oh.apply_transform_weight(w.double(), value.double(), location, module_type).bfloat16()
    _assert_within_ulp(got, want, f"{location} {module_type.__name__}")


@pytest.mark.parametrize("b", [32, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matrix_core_kernel_with_a_224_block(b, dtype, ctmi, gpu, hadamard_blocks):
    """ctmi_hadamard_apply for 224 x 32 and 224 x 64 (7168, 14336) straight through the C ABI:
    x diag(s_in) (Ma (x) Sylvester(b)) diag(s_out) / sqrt(n) against fp64, Ma the known
    Hadamard matrix of order 224 and a random +-1 matrix; more rows than workgroups hold at
    a time, and a count that leaves the last workgroup's waves without a row"""
    from compressed_tensors_amd import _lib

    announce("hadamard_apply 224 x", b, dtype)
    n = 224 * b
    g = torch.Generator().manual_seed(b)
    rows = 1027
    x = torch.randn(rows, n, generator=g).to(dtype)
    s_in = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    s_out = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    mb = oh.deterministic_hadamard_matrix(b, torch.bfloat16).to(gpu)
    sample = torch.tensor([0, 1, 255, 256, 511, 1023, 1024, 1026])
    for ma in (hadamard_blocks[224].double(), (torch.randint(0, 2, (224, 224), generator=g) * 2 - 1).double()):
        dense = torch.kron(ma, oh.deterministic_hadamard_matrix(b, torch.float64))
        ma_t = ma.T.contiguous().bfloat16().to(gpu)
        xg = x.to(gpu)
        for si, so in ((None, None), (s_in, None), (None, s_out)):
            out = torch.empty_like(xg)
            sig, sog = (None if t is None else t.to(gpu) for t in (si, so))
            _lib.check(ctmi.ctmi_hadamard_apply(xg.data_ptr(), out.data_ptr(), _lib.dtype_code(dtype), xg.numel(),
                                                224, b, ma_t.data_ptr(), mb.data_ptr(), _lib.ptr(sig),
                                                _lib.ptr(sog), _lib.stream_of(gpu)))
            xs = x[sample].double() * (1.0 if si is None else si.double())
            want = xs @ dense * (1.0 if so is None else so.double()) / n ** 0.5
            _assert_within_ulp(out[sample.to(gpu)], want.to(dtype), f"signs in={si is not None} out={so is not None}")
    assert ctmi.ctmi_hadamard_supported(224, 64, _lib.dtype_code(torch.float32)) == 0
    assert ctmi.ctmi_hadamard_supported(224, 128, _lib.dtype_code(torch.bfloat16)) == 0


@pytest.mark.parametrize("k,dtype,inner",
                         [(k, torch.bfloat16, 64) for k in (224, 12, 28, 36, 64, 100, 128, 160)] +
                         [(k, torch.float16, 64) for k in (224, 28, 64, 100)] +
                         [(k, torch.bfloat16, 32) for k in (224, 28, 64, 100, 128)] + [(224, torch.float16, 32)] +
                         [(k, torch.bfloat16, 128) for k in (224, 28, 64, 100, 128)] + [(224, torch.float16, 128)] +
                         [(k, torch.bfloat16, 16) for k in (224, 192, 28, 64, 100)] + [(224, torch.float16, 16)] +
                         [(k, torch.bfloat16, 8) for k in (224, 192, 20, 100)] + [(192, torch.float16, 8)] +
                         [(k, torch.bfloat16, 4) for k in (224, 192, 100, 240)] + [(224, torch.float16, 4)] +
                         [(160, torch.bfloat16, 128), (192, torch.bfloat16, 128), (148, torch.float16, 128),
                          (192, torch.bfloat16, 64), (148, torch.bfloat16, 32)] +
                         [(256, torch.bfloat16, 64), (240, torch.bfloat16, 64), (228, torch.bfloat16, 32),
                          (240, torch.bfloat16, 16), (252, torch.bfloat16, 8), (240, torch.float16, 64)],
                         ids=lambda v: str(v).replace("torch.", ""))
def test_block_times_sylvester64_with_butterflies(k, dtype, inner, ctmi, gpu, hadamard_blocks):
    """ctmi_hadamard_apply without mb_t (Mb = Sylvester(64)): the product with the block on the
    matrix cores, the Sylvester factor as butterflies on its fp32 result; bfloat16 and float16
    tensors (the block is given in bfloat16 either way); Sylvester(32), (16), (8) and (4) in place of
    Sylvester(64) (two, four, eight or sixteen runs share the kernel's 64 columns; numbers of runs that
    leave the last unit part empty, units that straddle the tensors of one call: 3584 = 224 * 16
    and 3072 = 192 * 16 are how the reference builds those sizes) and Sylvester(128) (28672 = 224 * 128: two halves of 64 columns and a
    stage over the halves).  Blocks of 228 ... 256 rows (15360 = 240 * 64, 3840 = 240 * 16) take two
    launches of four output tiles each and are refused in place.  Blocks of every tile
    count (K <= 32, 64, 128, 224) incl. sizes that leave rows of the last tile empty, a random
    +-1 matrix and (where the table has one) the known Hadamard block; more runs than the
    workgroups hold at a time; signs on either side; several tensors in one call."""
    from compressed_tensors_amd import _lib

    announce("block x Sylvester(4 ... 128), butterflies", k, dtype, inner)
    code = _lib.dtype_code(dtype)
    assert ctmi.ctmi_hadamard_sylvester_inner_supported(k, inner, code) == 1
    n = k * inner
    g = torch.Generator().manual_seed(k)
    rows = 2051 if k <= 64 else 1027
    if inner < 32:
        rows = 4 * rows + 1  # short runs: as many elements, and a last unit with one run
    x = torch.randn(rows, n, generator=g).to(dtype)
    s = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    sample = torch.tensor([0, 1, 255, 256, 511, 1023, 1024, rows - 1])
    blocks = [(torch.randint(0, 2, (k, k), generator=g) * 2 - 1).double()]
    if k in hadamard_blocks:
        blocks.append(hadamard_blocks[k].double())
    xg = x.to(gpu)
    for ma in blocks:
        sylvester = oh.deterministic_hadamard_matrix(inner, torch.float64)
        ma_t = ma.T.contiguous().bfloat16().to(gpu)
        for si, so in ((None, None), (s, None), (None, s)):
            out = torch.full_like(xg, float("nan"))
            sig, sog = (None if t is None else t.to(gpu) for t in (si, so))
            _lib.check(ctmi.ctmi_hadamard_apply(xg.data_ptr(), out.data_ptr(), code, xg.numel(), k, inner,
                                                ma_t.data_ptr(), None, _lib.ptr(sig), _lib.ptr(sog),
                                                _lib.stream_of(gpu)))
            assert not bool(torch.isnan(out.float()).any()), "every element written"
            xs = x[sample].double() * (1.0 if si is None else si.double())
            # x (Ma (x) S) for the run seen as a k x inner matrix X: Ma^T X S
            want = torch.einsum("rki,kj,im->rjm", xs.unflatten(-1, (k, inner)), ma, sylvester).flatten(-2, -1)
            want = want * (1.0 if so is None else so.double()) / n ** 0.5
            _assert_within_ulp(out[sample.to(gpu)], want.to(dtype), f"signs in={si is not None} out={so is not None}")
    # several tensors from one call == one by one
    ma_t = blocks[0].T.contiguous().bfloat16().to(gpu)
    xs = [torch.randn(r, n, generator=g).to(dtype).to(gpu) for r in (3, 70, 1, 16, 5, 9, 33, 2, 40, 7)]
    outs = [torch.empty_like(t) for t in xs]
    jobs = (_lib.HadamardJob * len(xs))()
    for job, t, o in zip(jobs, xs, outs):
        job.x, job.out, job.numel = t.data_ptr(), o.data_ptr(), t.numel()
    sg = s.to(gpu)
    _lib.check(ctmi.ctmi_hadamard_apply_many(jobs, len(xs), code, k, inner, ma_t.data_ptr(), None, sg.data_ptr(), None,
                                             _lib.stream_of(gpu)))
    for t, o in zip(xs, outs):
        one = torch.empty_like(t)
        _lib.check(ctmi.ctmi_hadamard_apply(t.data_ptr(), one.data_ptr(), code, t.numel(), k, inner, ma_t.data_ptr(),
                                            None, sg.data_ptr(), None, _lib.stream_of(gpu)))
        assert_bit_equal(o, one, f"tensor of {t.shape[0]} runs")
    # what it does not take
    assert ctmi.ctmi_hadamard_sylvester_inner_supported(k, 256, code) == 0
    assert ctmi.ctmi_hadamard_sylvester_inner_supported(257, 64, code) == 0
    assert ctmi.ctmi_hadamard_sylvester_inner_supported(225, 128, code) == 0
    if k > 224:
        rc = ctmi.ctmi_hadamard_apply(xg.data_ptr(), xg.data_ptr(), code, xg.numel(), k, inner, ma_t.data_ptr(), None,
                                      sg.data_ptr(), None, _lib.stream_of(gpu))
        assert rc == _lib.CTMI_ERR_VALUE  # the second launch would read what the first wrote
    assert ctmi.ctmi_hadamard_sylvester_inner_supported(k, 64, _lib.dtype_code(torch.float32)) == 0
    rc = ctmi.ctmi_hadamard_apply(xg.data_ptr(), xg.data_ptr(), code, xg.numel(), k, inner, ma_t.data_ptr(), None,
                                  sg.data_ptr(), sg.data_ptr(), _lib.stream_of(gpu))
    assert rc == _lib.CTMI_ERR_UNSUPPORTED


def test_zz_report_elements_beyond_one_ulp():
    """runs last in this file: the share of compared 16-bit outputs that differed from the
    fp64 result by more than one ulp of the output dtype (and passed on the allowance for
    fp32 accumulation, 2^-21 of the row's largest magnitude)"""
    n, k = ALLOWANCE["elements"], ALLOWANCE["leaning"]
    print(f"[hadamard] {k} of {n} compared 16-bit elements were more than 1 ulp off ({k / max(n, 1):.2e})", flush=True)
    assert k <= 1e-4 * max(n, 1)
