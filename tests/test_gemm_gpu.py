"""GEMM parity on the GPU, through the C ABI, against the CPU oracle on the same
seeded inputs.  Tolerance for half precision: 2e-2*sqrt(K)/sqrt(1024), scaled by
max(1,|ref|); fp32: 1e-4 relative to the float64 product."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_bf16, round_f16, tol_for_k, tol_half

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t.to(dtype) if dtype is not None else t


def test_fp32_1024_matches_cpu_packed_path(tracea_gpu):
    # configuration 1: M=N=K=1024, U[-1,1) from seed; the device result is compared with the
    # restated gemm_cpu_packed (hero tiling) and with the float64 product
    rng = np.random.default_rng(0x7ACEA001)
    a = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    b = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    c = tracea_gpu.gemm(_dev(a), _dev(b)).cpu().numpy()
    ref64 = oracle.gemm_f64(a, b)
    assert np.abs(c - ref64).max() <= 1e-4 * np.abs(ref64).max()
    packed = np.zeros((1024, 1024), np.float32)
    oracle.gemm_cpu_packed(a, b, packed)
    assert np.abs(c - packed).max() <= 2e-4 * np.abs(ref64).max()
    # all-ones variant of examples/cpu_bench.rs: exactly K everywhere
    ones = torch.ones(1024, 1024, device="cuda")
    assert (tracea_gpu.gemm(ones, ones) == 1024).all().item()


# fp32 kernels by shape: the 64x64 tile (few large tiles: the first two, (200, 300, 1000) split three
# ways along K, (1000, 1000, 40) with a ragged last K tile and an odd tile count), the 128x128 tile
# (2047 x 2044: 256 large tiles, one per CU), the any-layout kernel (N not a multiple of 4)
# (K tiles of 32 for launches of at most one workgroup per CU: (512, 512, 1040) with half a K tile at the
# end and four K ranges of an odd number of 16-wide tiles, (1024, 1024, 1072) unsplit, (320, 256, 2064) split)
@pytest.mark.parametrize("shape", [(64, 64, 64), (100, 36, 52), (129, 257, 200), (5, 4, 8), (200, 300, 1000),
                                   (1000, 1000, 40), (2047, 2044, 72), (192, 64, 16), (65, 68, 4),
                                   (512, 512, 1040), (1024, 1024, 1072), (320, 256, 2064), (768, 1024, 1040)])
def test_fp32_edges_and_fallback(tracea_gpu, shape):
    m, n, k = shape
    rng = np.random.default_rng(m * 7 + n)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    c = tracea_gpu.gemm(_dev(a), _dev(b)).cpu().numpy()
    ref = oracle.gemm_f64(a, b)
    assert np.abs(c - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())


def test_reference_known_answer_16cubed_f16(tracea_gpu):
    # tests/numerical_parity.rs:62-151: the reference's only numeric GPU test, tolerance 5e-2
    a = (np.arange(256, dtype=np.float32) * np.float32(0.05) - np.float32(0.4)).reshape(16, 16)
    b = (np.arange(256, dtype=np.float32) * np.float32(0.02) - np.float32(0.1)).reshape(16, 16)
    ref = oracle.gemm_f64(round_f16(a), round_f16(b))
    c = tracea_gpu.gemm(_dev(a, torch.float16), _dev(b, torch.float16)).float().cpu().numpy()
    # entries reach ~500, where one f16 step is 0.25: the reference's absolute 5e-2 can only hold
    # below 64; beyond that the f16 output rounding (relative 2^-11) is the floor
    small = np.abs(ref) < 64
    assert np.abs(c - ref)[small].max() < 5e-2
    assert_close_scaled(c, ref, 2.0 ** -10, "16^3 known answer")


HALF_SHAPES = [(256, 256, 128), (300, 200, 136), (512, 384, 1024), (64, 72, 8), (1000, 24, 72)]


@pytest.mark.parametrize("variant", range(40))
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_half_every_variant_both_b_layouts(tracea_gpu, variant, dtype):
    from tracea_amd import capi
    names = capi.variants("gemm")
    if variant >= len(names):
        pytest.skip("no such variant")
    tdt, rnd = (torch.float16, round_f16) if dtype == "f16" else (torch.bfloat16, round_bf16)
    capi.force_variant("gemm", variant)
    try:
        for (m, n, k) in HALF_SHAPES:
            rng = np.random.default_rng(1000 * variant + m + n + k)
            a = rnd(rng.standard_normal((m, k)) / np.sqrt(k))
            bt = rnd(rng.standard_normal((n, k)))          # column-major B: stored [N,K]
            ref = oracle.gemm_f64(a, bt.T)
            da, dbt = _dev(a, tdt), _dev(bt, tdt)
            c = tracea_gpu.gemm(da, dbt.t()).float().cpu().numpy()
            assert_close_scaled(c, ref, tol_half(k, dtype), "%s %s NT %s" % (names[variant], dtype, (m, n, k)))
            c2 = tracea_gpu.gemm(da, dbt.t().contiguous()).float().cpu().numpy()  # row-major B [K,N]
            assert_close_scaled(c2, ref, tol_half(k, dtype), "%s %s NN %s" % (names[variant], dtype, (m, n, k)))
    finally:
        capi.force_variant("gemm", -1)


def test_members_on_16x16x32_mfmas(tracea_gpu):
    """The MFMA shape is an axis of the family: the _m16 members multiply with v_mfma_f32_16x16x32, for both
    layouts of B, and agree with the oracle and with their 32x32x16 twins (in practice bit for bit)."""
    from tracea_amd import capi
    names = capi.variants("gemm")
    m16 = [nm for nm in names if nm.endswith("_m16")]
    assert len(m16) >= 3
    rng = np.random.default_rng(16)
    try:
        for (m, n, k) in [(520, 392, 1088), (256, 512, 192), (100, 72, 2048)]:   # ragged M and N, 17 / 3 / 32 K tiles
            a = round_f16(rng.standard_normal((m, k)) / np.sqrt(k))
            bt = round_f16(rng.standard_normal((n, k)))
            ref = oracle.gemm_f64(a, bt.T)
            da, dbt = _dev(a, torch.float16), _dev(bt, torch.float16)
            for nm in m16:
                twin = nm[: -len("_m16")]
                assert twin in names
                for b in (dbt.t(), dbt.t().contiguous()):          # K-contiguous and N-contiguous B
                    capi.force_variant("gemm", nm)
                    c = tracea_gpu.gemm(da, b)
                    assert capi.last_variant("gemm") == nm
                    assert_close_scaled(c.float().cpu().numpy(), ref, tol_half(k, "f16"), "%s %s" % (nm, (m, n, k)))
                    capi.force_variant("gemm", twin)
                    c_t = tracea_gpu.gemm(da, b)
                    assert_close_scaled(c.float().cpu().numpy(), c_t.float().cpu().numpy(), 2.0 ** -10, nm + " vs twin")
    finally:
        capi.force_variant("gemm", -1)
    # the default for a large product is a 16x16x32 member: four waves for a K-contiguous B, eight for an
    # N-contiguous one (twice the B fragments per wave on four)
    big = torch.randn(4096, 4096, device="cuda").half()
    wide = torch.randn(4096, 4096, device="cuda").half()
    tracea_gpu.gemm(big, wide.t())
    assert capi.last_variant("gemm") == "t256x256x64_w2x2_p2_m16"
    tracea_gpu.gemm(big, wide.t().contiguous())
    assert capi.last_variant("gemm") == "t256x256x64_w2x4_p2_m16"


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_tiles_stored_from_registers_equal_the_staged_rows(tracea_gpu, dtype):
    """With an empty chain the four-wave members on 16x16x32 MFMAs store a tile from registers (a lane swap
    per packed register pair) instead of staging it in LDS.  Adding a bias of zeros forces the staged rows:
    the two outputs must be equal element for element, on full tiles, on a tile cut by the end of M, and on
    both layouts of B."""
    from tracea_amd import capi
    tdt, rnd = (torch.float16, round_f16) if dtype == "f16" else (torch.bfloat16, round_bf16)
    names = capi.variants("gemm")
    members = [nm for nm in names if nm.endswith("_m16") and "w2x4" not in nm]
    assert members
    rng = np.random.default_rng(5)
    try:
        for (m, n, k) in [(512, 512, 320), (300, 768, 200)]:
            a = _dev(rnd(rng.standard_normal((m, k)) / np.sqrt(k)), tdt)
            bt = _dev(rnd(rng.standard_normal((n, k))), tdt)
            zeros = torch.zeros(n, device="cuda", dtype=torch.float32)
            ref = oracle.gemm_f64(a.float().cpu().numpy(), bt.float().cpu().numpy().T)
            for nm in members:
                capi.force_variant("gemm", nm)
                for b in (bt.t(), bt.t().contiguous()):
                    plain = tracea_gpu.gemm(a, b)
                    assert capi.last_variant("gemm") == nm
                    staged = tracea_gpu.gemm_ex(a, b, [(capi.OP_BIAS_ADD, zeros)])
                    assert torch.equal(plain, staged), "%s (%d, %d, %d)" % (nm, m, n, k)
                    assert_close_scaled(plain.float().cpu().numpy(), ref, tol_half(k, dtype), nm)
    finally:
        capi.force_variant("gemm", -1)


def test_epilogue_kinds_match_oracle_chain(tracea_gpu):
    # operator order of src/interface/c_bindings.rs:144-197, functors of epilogue.cuh
    m, n, k = 256, 320, 256
    rng = np.random.default_rng(77)
    a = round_f16(rng.standard_normal((m, k)) / np.sqrt(k))
    bt = round_f16(rng.standard_normal((n, k)))
    bias = rng.standard_normal(n).astype(np.float32)
    res = round_f16(rng.standard_normal((m, n)))
    acc = oracle.gemm_f64(a, bt.T).astype(np.float32)
    da, dbt = _dev(a, torch.float16), _dev(bt, torch.float16)
    dbias, dres = _dev(bias), _dev(res, torch.float16)
    E = oracle
    cases = {
        "none": [],
        "bias": [(E.EPI_BIAS_ADD, bias)],
        "relu": [(E.EPI_RELU,)],
        "gelu": [(E.EPI_GELU,)],
        "silu": [(E.EPI_SILU,)],
        "bias+relu": [(E.EPI_BIAS_ADD, bias), (E.EPI_RELU,)],
        "bias+silu": [(E.EPI_BIAS_ADD_SILU, bias)],
        "residual": [(E.EPI_RESIDUAL_ADD, res)],
        "residual+relu": [(E.EPI_RESIDUAL_ADD, res), (E.EPI_RELU,)],
    }
    for name, chain in cases.items():
        want = oracle.epilogue_apply(acc, chain)
        got = tracea_gpu.gemm(da, dbt.t(), bias=dbias if "bias" in name else None,
                              residual=dres if "residual" in name else None,
                              epilogue=name).float().cpu().numpy()
        assert_close_scaled(got, want, tol_for_k(k), "epilogue " + name)
    # f16 bias and fp32 output
    got = tracea_gpu.gemm(da, dbt.t(), bias=_dev(bias, torch.float16), epilogue="bias",
                          out_dtype=torch.float32).cpu().numpy()
    want = oracle.epilogue_apply(acc, [(E.EPI_BIAS_ADD, round_f16(bias))])
    assert_close_scaled(got, want, 1e-3, "f16 bias, f32 out")


def test_explicit_chain_with_batchnorm(tracea_gpu):
    from tracea_amd import capi
    m, n, k = 128, 64, 64
    rng = np.random.default_rng(5)
    a = round_f16(rng.standard_normal((m, k)) / np.sqrt(k))
    bt = round_f16(rng.standard_normal((n, k)))
    gamma = rng.uniform(0.5, 1.5, n).astype(np.float32)
    beta = (rng.standard_normal(n) * 0.1).astype(np.float32)
    mean = (rng.standard_normal(n) * 0.1).astype(np.float32)
    var = rng.uniform(0.5, 1.5, n).astype(np.float32)
    acc = oracle.gemm_f64(a, bt.T).astype(np.float32)
    want = oracle.epilogue_apply(acc, [(oracle.EPI_BATCHNORM, gamma, beta, mean, var, 1e-5), (oracle.EPI_RELU,)])
    got = tracea_gpu.gemm_ex(_dev(a, torch.float16), _dev(bt, torch.float16).t(),
                             [(capi.OP_BATCHNORM, _dev(gamma), _dev(beta), _dev(mean), _dev(var), 1e-5),
                              (capi.OP_RELU,)]).float().cpu().numpy()
    assert_close_scaled(got, want, tol_for_k(k), "BN+ReLU chain")


@pytest.mark.parametrize("shape", [(4096, 4096, 4096), (8192, 2048, 8192)])
def test_full_size_fp16_sampled_rows_and_linearity(tracea_gpu, shape):
    # configuration 2 at its real size: N(0,1)/sqrt(K) entries, A row-major, B column-major.
    # 48 sampled rows are checked against the float64 oracle; the whole output is checked
    # through linearity: gemm(A, B)[rows] == gemm(A[rows], B) bit for bit (same kernel, same
    # per-row arithmetic) and gemm(2A, B) == 2 gemm(A, B) exactly (powers of two commute with rounding).
    m, n, k = shape
    g = torch.Generator(device="cuda").manual_seed(0x7ACEA002)
    a = (torch.randn(m, k, device="cuda", generator=g) / k ** 0.5).half()
    bt = (torch.randn(n, k, device="cuda", generator=g) / k ** 0.5).half()
    c = tracea_gpu.gemm(a, bt.t())
    rows = np.random.default_rng(1).choice(m, 48, replace=False)
    ref = oracle.gemm_f64(a[rows].float().cpu().numpy(), bt.float().cpu().numpy().T)
    assert_close_scaled(c[rows].float().cpu().numpy(), ref, tol_for_k(k), "sampled rows %s" % (shape,))
    c2 = tracea_gpu.gemm(a * 2, bt.t())
    normal = c.float().abs() >= 2.0 ** -13   # f16 rounding is scale-invariant only for normal numbers
    assert torch.equal(c2[normal], (c * 2)[normal])
    assert ((c2.float() - 2 * c.float()).abs() <= 2.0 ** -23).all().item()  # subnormal outputs: one step
    assert torch.isfinite(c.float()).all().item()


def test_error_paths(tracea_gpu):
    from tracea_amd import capi
    a = torch.zeros(8, 8, device="cuda", dtype=torch.float16)
    with pytest.raises(capi.TraceaError) as e:
        tracea_gpu.gemm(a, torch.zeros(16, 8, device="cuda", dtype=torch.float16))
    assert e.value.status == capi.INVALID_PARAMS
    with pytest.raises(capi.TraceaError) as e:
        tracea_gpu.gemm(a.int(), a.int(), out=a.int())
    assert e.value.status == capi.UNSUPPORTED_CONFIG
    host = torch.zeros(8, 8, dtype=torch.float16)
    with pytest.raises(capi.TraceaError) as e:
        tracea_gpu.gemm(host, host, out=host.clone())
    assert e.value.status == capi.CPU_ERROR
    with pytest.raises(capi.TraceaError) as e:
        tracea_gpu.gemm(a, a, bias=torch.zeros(7, device="cuda"), epilogue="bias")
    assert e.value.status == capi.INVALID_PARAMS
    # NULL data pointer
    shape = (C.c_uint64 * 2)(8, 8)
    tv = capi.TensorView(None, 2, shape, None, capi.F16, 0)
    st = capi.lib().tracea_gemm(tv, tv, None, None, C.byref(tv), capi.GemmParams(0, None))
    assert st == capi.INVALID_PARAMS


def test_half_precision_batchnorm_parameters_are_refused(tracea_gpu):
    # the kernels read BatchNorm / scale-shift vectors as fp32: the library refuses an operator
    # that names another type (straight through the C ABI, past the Python wrapper's own check)
    from tracea_amd import capi
    from tracea_amd import ops as raw
    a = torch.zeros(64, 64, device="cuda", dtype=torch.float16)
    out = torch.empty(64, 64, device="cuda", dtype=torch.float16)
    vec = torch.ones(64, device="cuda", dtype=torch.float16)
    for kind, n_tensors in ((capi.OP_BATCHNORM, 4), (capi.OP_SCALE_SHIFT, 2)):
        arr = (capi.EpilogueOp * 1)()
        arr[0].kind = kind
        arr[0].dtype = capi.F16
        for slot in ("p0", "p1", "p2", "p3")[:n_tensors]:
            setattr(arr[0], slot, vec.data_ptr())
        arr[0].epsilon = 1e-5
        va, vb, vc = raw._view(a), raw._view(a.t()), raw._view(out)
        st = capi.lib().tracea_gemm_ex(va.c, vb.c, C.byref(vc.c), capi.GemmParams(0, None), arr, 1)
        assert st == capi.UNSUPPORTED_CONFIG
        assert "float32" in capi.last_error()
    with pytest.raises(ValueError):
        tracea_gpu.gemm_ex(a, a.t(), [(capi.OP_SCALE_SHIFT, vec, vec)])


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_operand_beyond_2gib_takes_the_register_staged_kernels(tracea_gpu, dtype):
    # the direct-to-LDS kernels address operands with 32-bit byte offsets; an A whose rows are spread
    # over more than 2 GiB must run on the kernels that form 64-bit addresses, with the same results
    from tracea_amd import capi
    m, n, k = 130, 200, 192
    tdt = torch.float32 if dtype == "f32" else torch.float16
    lda = (2 ** 31 // (m - 1)) // tdt.itemsize + 64          # (m-1)*lda*itemsize just above 2 GiB
    lda -= lda % 8
    buf = torch.empty((m - 1) * lda + k, dtype=tdt, device="cuda")
    a_view = buf.as_strided((m, k), (lda, 1))
    assert ((m - 1) * lda + k) * tdt.itemsize >= 2 ** 31
    rng = np.random.default_rng(77)
    a = (rng.standard_normal((m, k)) / np.sqrt(k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    if dtype == "f16":
        a, b = round_f16(a), round_f16(b)
    a_view.copy_(_dev(a, tdt))
    bias = rng.standard_normal(n).astype(np.float32)
    got = tracea_gpu.gemm(a_view, _dev(b, tdt), bias=_dev(bias), epilogue="bias+relu").float().cpu().numpy()
    ref = np.maximum(oracle.gemm_f64(a, b) + bias[None, :], 0.0)
    if dtype == "f32":
        assert np.abs(got - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
    else:
        name = capi.last_variant("gemm")
        assert "_p2" not in name and "_p3" not in name, name
        assert_close_scaled(got, ref, tol_half(k, "f16"), "A beyond 2 GiB")
    # the same product from a compact copy of A runs the direct-to-LDS kernels and agrees
    compact = tracea_gpu.gemm(a_view.contiguous(), _dev(b, tdt), bias=_dev(bias), epilogue="bias+relu").float().cpu().numpy()
    np.testing.assert_allclose(got, compact, rtol=0, atol=2e-3 if dtype == "f16" else 1e-5)


@pytest.mark.parametrize("shape", [(1000, 900, 1030), (129, 257, 203), (5, 3, 7), (300, 1001, 130), (1, 1, 1), (513, 130, 31)])
def test_ragged_sizes_and_strided_operands_run_from_padded_copies(tracea_gpu, shape):
    """A K or N that is not a whole number of 16-byte pieces, and operands strided along K: copied into padded rows
    and multiplied by the tile kernels (the any-layout kernel on the vector ALU remains for what cannot be copied).
    fp32 and both half types, B row-major and column-major, a column-major A, with a chain and with fp32 output."""
    from tracea_amd import capi
    m, n, k = shape
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a = (rng.standard_normal((m, k)) / np.sqrt(k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    ref = np.maximum(oracle.gemm_f64(a, b) + bias[None, :], 0.0)
    da, db, dbias = _dev(a), _dev(b), _dev(bias)
    for tag, xa, xb in (("row-major B", da, db), ("column-major B", da, db.t().contiguous().t()),
                        ("column-major A", da.t().contiguous().t(), db)):
        got = tracea_gpu.gemm(xa, xb, bias=dbias, epilogue="bias+relu").cpu().numpy()
        assert np.abs(got - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max()), "f32 " + tag
    for dtype, tdt, rnd in (("f16", torch.float16, round_f16), ("bf16", torch.bfloat16, round_bf16)):
        ha, hb = rnd(a), rnd(b)
        ref16 = oracle.gemm_f64(ha, hb)
        want = np.maximum(ref16 + bias[None, :], 0.0)
        xa, xb = _dev(ha, tdt), _dev(hb, tdt)
        for tag, yb in (("row-major B", xb), ("column-major B", xb.t().contiguous().t())):
            got = tracea_gpu.gemm(xa, yb, bias=dbias, epilogue="bias+relu").float().cpu().numpy()
            assert capi.last_variant("gemm") is not None, "the tile kernels did not run"
            assert_close_scaled(got, want, tol_half(k, dtype), "%s %s" % (dtype, tag))
        got = tracea_gpu.gemm(xa, xb, out_dtype=torch.float32).cpu().numpy()
        assert np.abs(got - ref16).max() <= 1e-4 * max(1.0, np.abs(ref16).max()), dtype + " with fp32 output"
