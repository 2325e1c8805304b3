"""Parity of each HIP kernel, called through the C ABI, against the numpy oracle."""
import numpy as np
import pytest
import torch

from oracle import ops as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from poptransformer_amd import kernels
    return kernels


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def rel_err(got, ref):
    got = got.astype(np.float64)
    ref = ref.astype(np.float64)
    return np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30)


# ---------------------------------------------------------------- Int4ToHalf (bit-exact)
@pytest.mark.parametrize("n,m", [(3, 2), (16, 64), (130, 70), (11008, 64)])
@pytest.mark.parametrize("axis", [0, 1])
def test_int4_to_half_bit_exact(K, n, m, axis):
    rng = np.random.default_rng(n * 131 + m + axis)
    packed = rng.integers(-128, 128, size=(n, m), dtype=np.int8)
    scale = rng.uniform(0.005, 0.02, size=(n if axis == 1 else m,)).astype(np.float16)
    got = host(K.int4_to_half(dev(packed), dev(scale), axis))
    ref = O.int4_to_half(packed, scale, axis)
    assert got.shape == ref.shape
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


def test_int4_to_half_all_bytes(K):
    packed = np.arange(256, dtype=np.uint8).view(np.int8).reshape(256, 1)
    scale = np.ones(256, np.float16)
    got = host(K.int4_to_half(dev(packed), dev(scale), 1))        # [2, 256]
    tab = O.int4_table()
    assert np.array_equal(got.T.astype(np.float32), tab)


def test_int4_to_half_guards(K):
    p = dev(np.zeros((4, 4), np.int8))
    s = dev(np.ones(4, np.float16))
    with pytest.raises(ValueError):
        K.int4_to_half(p, s, axis=2)
    with pytest.raises(ValueError):
        K.int4_to_half(p, dev(np.ones(5, np.float16)), axis=1)
    with pytest.raises(ValueError):
        K.int4_to_half(dev(np.zeros((4,), np.int8)), s, axis=1)


# ---------------------------------------------------------------- W4A16 GEMM
def _w4_case(seed, M, Kdim, N):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    packed = rng.integers(-128, 128, size=(N, Kdim // 2), dtype=np.int8)
    scale = rng.uniform(0.005, 0.02, size=(N,)).astype(np.float16)
    return x, packed, scale


@pytest.mark.parametrize("M", [1, 4, 16, 17, 33, 64])
@pytest.mark.parametrize("Kdim,N", [(128, 16), (256, 48), (1024, 100), (4096, 512), (11008, 64), (136, 24)])
def test_w4a16_gemm(K, M, Kdim, N):
    x, packed, scale = _w4_case(M * 7 + Kdim + N, M, Kdim, N)
    w = K.W4Weight(dev(packed), dev(scale))
    got = host(K.w4a16_gemm(dev(x), w))
    ref64 = x.astype(np.float64) @ O.int4_to_half(packed, scale, 1).astype(np.float64)
    ref = O.w4a16_matmul(x, packed, scale)
    assert got.shape == ref.shape
    # north-star tolerance: max rel err <= 1e-2 on fp16 outputs
    assert rel_err(got, ref) <= 1e-2
    # against exact arithmetic the kernel must be as good as fp16 rounding allows
    assert np.abs(got.astype(np.float64) - ref64).max() <= 2.0 ** -10 * np.abs(ref64).max() + 1e-3


def test_w4a16_gemm_exact_integers(K):
    """Integers small enough that every product and sum is exact: the result must be exact,
    which catches any wrong nibble order, sign or feature permutation."""
    rng = np.random.default_rng(5)
    M, Kdim, N = 5, 256, 40
    x = rng.integers(-2, 3, size=(M, Kdim)).astype(np.float16)
    q = rng.integers(-8, 8, size=(N, Kdim))
    packed = O.pack_int4(q)
    scale = np.ones(N, np.float16)
    w = K.W4Weight(dev(packed), dev(scale))
    got = host(K.w4a16_gemm(dev(x), w)).astype(np.int64)
    ref = x.astype(np.int64) @ q.T.astype(np.int64)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("M", [17, 32, 33, 64])
@pytest.mark.parametrize("Kdim,N", [(1024, 8192), (1160, 4096), (4096, 8192)])
def test_w4a16_gemm_many_rows_wide_outputs(K, M, Kdim, N):
    """More than 16 rows and enough output channels to fill the machine: the kernel that stages the
    activation rows in LDS (4096 channels only up to 32 rows; 1160 features = a ragged last tile)."""
    x, packed, scale = _w4_case(M * 3 + Kdim + N, M, Kdim, N)
    w = K.W4Weight(dev(packed), dev(scale))
    got = host(K.w4a16_gemm(dev(x), w))
    ref = O.w4a16_matmul(x, packed, scale)
    assert rel_err(got, ref) <= 1e-2
    ref64 = x.astype(np.float64) @ O.int4_to_half(packed, scale, 1).astype(np.float64)
    assert np.abs(got.astype(np.float64) - ref64).max() <= 2.0 ** -10 * np.abs(ref64).max() + 1e-3


@pytest.mark.parametrize("M", [20, 33, 64])
def test_w4a16_gemm_many_rows_more_workgroups_than_compute_units(K, M):
    """17..64 rows and more than 256 workgroups of 64 channels: the launch takes workgroups of 16 waves and 128
    channels.  The two weights of the RWKV channel mix (16384 and 4096 channels, models/rwkv/ffn.py:
    47-56) with an input and an activation each, and one weight of 20480 channels with bias and residual; 1160
    features = a ragged last tile."""
    print(f"case: four streams per wave, {M} rows", flush=True)
    rng = np.random.default_rng(M)
    Kdim = 1160
    xs = [rng.standard_normal((M, Kdim)).astype(np.float16) for _ in range(2)]
    cases = [_w4_case(M + n, 1, Kdim, n)[1:] for n in (16384, 4096)]
    ws = [K.W4Weight(dev(p_), dev(s_)) for p_, s_ in cases]
    outs = [torch.empty((M, n), dtype=torch.float16, device="cuda") for n in (16384, 4096)]
    K.linear(None, ws, outs, xs=[dev(x) for x in xs], acts=[K._lib.ACT_RELU_SQUARE, K._lib.ACT_SIGMOID])
    ref0 = O.w4a16_matmul(xs[0], *cases[0]); ref0 = (np.maximum(ref0, np.float16(0)) ** 2).astype(np.float16)
    ref1 = O.w4a16_matmul(xs[1], *cases[1]).astype(np.float32); ref1 = (1.0 / (1.0 + np.exp(-ref1))).astype(np.float16)
    assert rel_err(host(outs[0]), ref0) <= 1e-2 and rel_err(host(outs[1]), ref1) <= 1e-2
    x, packed, scale = _w4_case(M * 5, M, Kdim, 20480)
    bias = rng.standard_normal(20480).astype(np.float16)
    res = rng.standard_normal((M, 20480)).astype(np.float16)
    got = host(K.w4a16_gemm(dev(x), K.W4Weight(dev(packed), dev(scale)), bias=dev(bias), residual=dev(res)))
    ref = ((O.w4a16_matmul(x, packed, scale) + bias).astype(np.float16) + res).astype(np.float16)
    assert rel_err(got, ref) <= 1e-2
    ref64 = x.astype(np.float64) @ O.int4_to_half(packed, scale, 1).astype(np.float64) + bias.astype(np.float64) + res.astype(np.float64)
    assert np.abs(got.astype(np.float64) - ref64).max() <= 3 * 2.0 ** -10 * np.abs(ref64).max() + 1e-3


@pytest.mark.parametrize("M", [17, 32, 33, 64])
@pytest.mark.parametrize("Kdim,N", [(4096, 1024), (11008, 4096), (2872, 2048)])
def test_w4a16_gemm_many_rows_few_outputs_split_k(K, M, Kdim, N):
    """More than 16 rows and too few output channels to fill the machine: with a workspace the launch also
    splits the features across workgroups (2872 features = 23 tiles, the last ragged: slices of unequal length)
    and a second kernel adds the slices and applies bias and residual.  Against the oracle, and against the
    launch without workspace (same sums in another order)."""
    x, packed, scale = _w4_case(M + Kdim + N, M, Kdim, N)
    rng = np.random.default_rng(M + N)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    w = K.W4Weight(dev(packed), dev(scale))
    ws = K.linear_workspace(M, N, "cuda")
    ws.fill_(0xFF)                                        # NaN patterns: every slice must be written before it is read
    y = dev(res.copy())
    K.w4a16_gemm(dev(x), w, bias=dev(bias), residual=y, out=y, workspace=ws)       # the residual aliases the output
    got = host(y)
    ref = ((O.w4a16_matmul(x, packed, scale) + bias).astype(np.float16) + res).astype(np.float16)
    assert rel_err(got, ref) <= 1e-2
    plain = host(K.w4a16_gemm(dev(x), w, bias=dev(bias), residual=dev(res)))
    assert rel_err(got, plain) <= 2e-3
    small = torch.empty(64, dtype=torch.uint8, device="cuda")                      # too small: the one-kernel form runs
    assert rel_err(host(K.w4a16_gemm(dev(x), w, bias=dev(bias), residual=dev(res), workspace=small)), ref) <= 1e-2
    # the gate and the halving of the RWKV channel mix (models/rwkv/ffn.py:58, model.py:115-116) behind the split
    gate = rng.uniform(0, 1, (M, N)).astype(np.float16)
    outs = []
    for wsp in (ws, None):
        y = dev(res.copy())
        K.linear(dev(x), [w], [y], mul=dev(gate), residual=y, post_scale=0.5, workspace=wsp)
        outs.append(host(y))
    want = (((O.w4a16_matmul(x, packed, scale) * gate).astype(np.float16) + res).astype(np.float16) * np.float16(0.5)).astype(np.float16)
    assert rel_err(outs[0], want) <= 1e-2 and rel_err(outs[0], outs[1]) <= 2e-3


def test_w4a16_gemm_many_rows_exact_integers(K):
    rng = np.random.default_rng(6)
    M, Kdim, N = 40, 1024, 8192
    x = rng.integers(-2, 3, size=(M, Kdim)).astype(np.float16)
    q = rng.integers(-8, 8, size=(N, Kdim))
    w = K.W4Weight(dev(O.pack_int4(q)), dev(np.ones(N, np.float16)))
    got = host(K.w4a16_gemm(dev(x), w)).astype(np.int64)
    assert np.array_equal(got, x.astype(np.int64) @ q.T.astype(np.int64))


def test_w4a16_gemm_many_rows_multi_swiglu_epilogue(K):
    rng = np.random.default_rng(8)
    M, Kdim = 33, 1024
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    mats = []
    for N in (4096, 2048, 2048):
        mats.append((rng.integers(-128, 128, size=(N, Kdim // 2), dtype=np.int8),
                     rng.uniform(0.005, 0.02, size=(N,)).astype(np.float16)))
    ws = [K.W4Weight(dev(p), dev(s)) for p, s in mats]
    for (p, s), o in zip(mats, K.w4a16_gemm_multi(dev(x), ws)):
        assert rel_err(host(o), O.w4a16_matmul(x, p, s)) <= 1e-2
    N = 8192
    (pg, sg), (pu, su) = [(rng.integers(-128, 128, size=(N, Kdim // 2), dtype=np.int8),
                           rng.uniform(0.005, 0.02, size=(N,)).astype(np.float16)) for _ in range(2)]
    got = host(K.w4a16_gemm_swiglu(dev(x), K.W4Weight(dev(pg), dev(sg)), K.W4Weight(dev(pu), dev(su))))
    ref = (O.w4a16_matmul(x, pu, su) * O.swish(O.w4a16_matmul(x, pg, sg))).astype(np.float16)
    assert rel_err(got, ref) <= 1e-2
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    got = host(K.w4a16_gemm(dev(x), K.W4Weight(dev(pg), dev(sg)), bias=dev(bias), residual=dev(res)))
    ref = ((O.w4a16_matmul(x, pg, sg) + bias).astype(np.float16) + res).astype(np.float16)
    assert rel_err(got, ref) <= 1e-2


@pytest.mark.parametrize("M", [5, 8, 16])
@pytest.mark.parametrize("Kdim,N", [(4096, 13696), (1160, 13690), (1024, 13696), (2176, 13696)])
def test_w4a16_gemv_uneven_rounds_of_workgroups(K, M, Kdim, N):
    """Up to 16 rows and a number of channel blocks (856) that the workgroups of the 16-wave kernel cover in uneven
    rounds: the kernel in which one workgroup per compute unit walks its share of the blocks.  1160 and 2176 features =
    a ragged last tile / a block of one, two and four steps; 13690 channels = a ragged last block; bias and a residual
    that aliases the output."""
    x, packed, scale = _w4_case(M + Kdim + N, M, Kdim, N)
    rng = np.random.default_rng(M * N)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    w = K.W4Weight(dev(packed), dev(scale))
    plain = O.w4a16_matmul(x, packed, scale)
    assert rel_err(host(K.w4a16_gemm(dev(x), w)), plain) <= 1e-2
    y = dev(res.copy())
    K.w4a16_gemm(dev(x), w, bias=dev(bias), residual=y, out=y)
    assert rel_err(host(y), ((plain + bias).astype(np.float16) + res).astype(np.float16)) <= 1e-2


def test_gemv_uneven_rounds_exact_integers_multi_swiglu_f16(K):
    """The same kernel: integers small enough for exact sums (any wrong tile, step or lane shows), three matrices of
    different widths with their biases in one launch, the SwiGLU pair, and fp16 weights."""
    rng = np.random.default_rng(21)
    M, Kdim, N = 16, 1024, 13696
    x = rng.integers(-1, 2, size=(M, Kdim)).astype(np.float16)
    q = rng.integers(-8, 8, size=(N, Kdim))
    w = K.W4Weight(dev(O.pack_int4(q)), dev(np.ones(N, np.float16)))
    assert np.array_equal(host(K.w4a16_gemm(dev(x), w)).astype(np.int64), x.astype(np.int64) @ q.T.astype(np.int64))
    M, Kdim = 7, 4096
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    mats = [(rng.integers(-128, 128, size=(n, Kdim // 2), dtype=np.int8), rng.uniform(0.005, 0.02, size=(n,)).astype(np.float16))
            for n in (4096, 9000, 520)]
    ws = [K.W4Weight(dev(p), dev(s)) for p, s in mats]
    biases = [rng.standard_normal(p.shape[0]).astype(np.float16) for p, _ in mats]
    outs = [torch.empty((M, p.shape[0]), dtype=torch.float16, device="cuda") for p, _ in mats]
    K.linear(dev(x), ws, outs, biases=[dev(b) for b in biases])
    for (p, s), b, o in zip(mats, biases, outs):
        assert rel_err(host(o), (O.w4a16_matmul(x, p, s) + b).astype(np.float16)) <= 1e-2
    (pg, sg), (pu, su) = [(rng.integers(-128, 128, size=(N, Kdim // 2), dtype=np.int8),
                           rng.uniform(0.005, 0.02, size=(N,)).astype(np.float16)) for _ in range(2)]
    got = host(K.w4a16_gemm_swiglu(dev(x), K.W4Weight(dev(pg), dev(sg)), K.W4Weight(dev(pu), dev(su))))
    assert rel_err(got, (O.w4a16_matmul(x, pu, su) * O.swish(O.w4a16_matmul(x, pg, sg))).astype(np.float16)) <= 1e-2
    wf = (rng.standard_normal((Kdim, N)) * 0.05).astype(np.float16)
    got = host(K.f16_gemm(dev(x), K.F16Weight(dev(np.ascontiguousarray(wf.T)))))
    ref64 = x.astype(np.float64) @ wf.astype(np.float64)
    assert np.abs(got.astype(np.float64) - ref64).max() <= 2.0 ** -10 * np.abs(ref64).max() + 1e-3


def test_w4a16_gemm_epilogue(K):
    x, packed, scale = _w4_case(11, 3, 512, 96)
    rng = np.random.default_rng(12)
    bias = rng.standard_normal(96).astype(np.float16)
    res = rng.standard_normal((3, 96)).astype(np.float16)
    w = K.W4Weight(dev(packed), dev(scale))
    got = host(K.w4a16_gemm(dev(x), w, bias=dev(bias), residual=dev(res)))
    y = O.w4a16_matmul(x, packed, scale)
    ref = ((y + bias).astype(np.float16) + res).astype(np.float16)
    assert rel_err(got, ref) <= 1e-2


def test_w4a16_gemm_multi_and_swiglu(K):
    rng = np.random.default_rng(3)
    M, Kdim = 2, 1024
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    mats = []
    for N in (256, 64, 80):
        packed = rng.integers(-128, 128, size=(N, Kdim // 2), dtype=np.int8)
        scale = rng.uniform(0.005, 0.02, size=(N,)).astype(np.float16)
        mats.append((packed, scale))
    ws = [K.W4Weight(dev(p), dev(s)) for p, s in mats]
    outs = K.w4a16_gemm_multi(dev(x), ws)
    for (p, s), o in zip(mats, outs):
        assert rel_err(host(o), O.w4a16_matmul(x, p, s)) <= 1e-2
    (pg, sg), (pu, su) = (mats[1], (rng.integers(-128, 128, size=(64, Kdim // 2), dtype=np.int8),
                                    rng.uniform(0.005, 0.02, size=(64,)).astype(np.float16)))
    got = host(K.w4a16_gemm_swiglu(dev(x), K.W4Weight(dev(pg), dev(sg)), K.W4Weight(dev(pu), dev(su))))
    gate = O.swish(O.w4a16_matmul(x, pg, sg))
    ref = (O.w4a16_matmul(x, pu, su) * gate).astype(np.float16)
    assert rel_err(got, ref) <= 1e-2


@pytest.mark.parametrize("M", [1, 3])
def test_gemm_fused_norms(K, M):
    """RMSNorm / NormCE applied inside the GEMM must equal the norm entry point followed by the GEMM."""
    x, packed, scale = _w4_case(21, M, 768, 96)
    rng = np.random.default_rng(22)
    g = rng.uniform(0.5, 1.5, 768).astype(np.float16)
    b = rng.standard_normal(768).astype(np.float16)
    w = K.W4Weight(dev(packed), dev(scale))
    xd, gd, bd = dev(x), dev(g), dev(b)
    two = host(K.w4a16_gemm(K.rmsnorm(xd, gd, 1e-5), w))
    one = host(K.w4a16_gemm(xd, w, norm=K.Norm(gd, None, 1e-5)))
    assert rel_err(one, two) <= 2e-3
    assert rel_err(one, O.w4a16_matmul(O.rms_norm(x, g, 1e-5), packed, scale)) <= 1e-2
    w16 = (rng.standard_normal((64, 768)) * 0.05).astype(np.float16)
    fw = K.F16Weight(dev(w16))
    two = host(K.f16_gemm(K.layer_norm_ce(xd, gd, bd, 1e-5), fw))
    one = host(K.f16_gemm(xd, fw, norm=K.Norm(gd, bd, 1e-5)))
    assert rel_err(one, two) <= 2e-3
    assert rel_err(one, O.matmul(O.layer_norm_ce(x, g, b, 1e-5, M, 1, 768), w16.T)) <= 1e-2
    with pytest.raises(NotImplementedError):
        K.w4a16_gemm(dev(np.zeros((16, 768), np.float16)), w, norm=K.Norm(gd, None, 1e-5))


@pytest.mark.parametrize("M", [5, 16])
@pytest.mark.parametrize("Kdim,N", [(1160, 96), (4096, 4096)])
def test_gemm_fused_norms_up_to_16_rows(K, M, Kdim, N):
    """5..16 rows: the norm inside the GEMM (row sums in a pass of their own over the fragments each wave
    loads anyway) equals the norm entry point followed by the GEMM; 1160 features end in a ragged tile."""
    x, packed, scale = _w4_case(31 + M, M, Kdim, N)
    rng = np.random.default_rng(23 + Kdim)
    g = rng.uniform(0.5, 1.5, Kdim).astype(np.float16)
    b = (rng.standard_normal(Kdim) * 0.1).astype(np.float16)
    w = K.W4Weight(dev(packed), dev(scale))
    xd, gd, bd = dev(x), dev(g), dev(b)
    two = host(K.w4a16_gemm(K.rmsnorm(xd, gd, 1e-5), w))
    one = host(K.w4a16_gemm(xd, w, norm=K.Norm(gd, None, 1e-5)))
    assert rel_err(one, two) <= 2e-3
    assert rel_err(one, O.w4a16_matmul(O.rms_norm(x, g, 1e-5), packed, scale)) <= 1e-2
    two = host(K.w4a16_gemm(K.layer_norm_ce(xd, gd, bd, 1e-5), w))
    one = host(K.w4a16_gemm(xd, w, norm=K.Norm(gd, bd, 1e-5)))
    assert rel_err(one, two) <= 2e-3
    assert rel_err(one, O.w4a16_matmul(O.layer_norm_ce(x, g, b, 1e-5, M, 1, Kdim), packed, scale)) <= 1e-2
    # a SwiGLU pair and several weights in one launch, each with the norm inside
    _, pu, su = _w4_case(77, M, Kdim, N)
    wu = K.W4Weight(dev(pu), dev(su))
    h = K.rmsnorm(xd, gd, 1e-5)
    assert rel_err(host(K.w4a16_gemm_swiglu(xd, w, wu, norm=K.Norm(gd, None, 1e-5))), host(K.w4a16_gemm_swiglu(h, w, wu))) <= 2e-3
    for o1, o2 in zip(K.w4a16_gemm_multi(xd, [w, wu], norm=K.Norm(gd, None, 1e-5)), K.w4a16_gemm_multi(h, [w, wu])):
        assert rel_err(host(o1), host(o2)) <= 2e-3


def test_w4a16_guards(K):
    x, packed, scale = _w4_case(1, 1, 128, 16)
    w = K.W4Weight(dev(packed), dev(scale))
    with pytest.raises(ValueError):
        K.w4a16_gemm(dev(np.zeros((1, 64), np.float16)), w)
    with pytest.raises(ValueError):
        K.w4a16_gemm(dev(np.zeros((4097, 128), np.float16)), w)


# ---------------------------------------------------------------- FP16 GEMM
@pytest.mark.parametrize("M,Kdim,N", [(1, 768, 50257), (4, 4096, 1000), (16, 128, 16), (64, 3072, 768), (1, 136, 20)])
def test_f16_gemm(K, M, Kdim, N):
    rng = np.random.default_rng(M + Kdim + N)
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    w = (rng.standard_normal((N, Kdim)) * 0.02).astype(np.float16)
    got = host(K.f16_gemm(dev(x), K.F16Weight(dev(w))))
    ref = O.matmul(x, w.T)
    assert rel_err(got, ref) <= 1e-2
    ref64 = x.astype(np.float64) @ w.T.astype(np.float64)
    assert np.abs(got.astype(np.float64) - ref64).max() <= 2.0 ** -10 * np.abs(ref64).max() + 1e-4


def test_f16_gemm_many_rows_wide_outputs(K):
    rng = np.random.default_rng(21)
    M, Kdim, N = 24, 1024, 8192
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    w = (rng.standard_normal((N, Kdim)) * 0.02).astype(np.float16)
    got = host(K.f16_gemm(dev(x), K.F16Weight(dev(w))))
    assert rel_err(got, O.matmul(x, w.T)) <= 1e-2


def test_f16_gemm_gelu_bias(K):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((2, 256)).astype(np.float16)
    w = (rng.standard_normal((64, 256)) * 0.05).astype(np.float16)
    b = rng.standard_normal(64).astype(np.float16)
    from poptransformer_amd import _lib
    got = host(K.f16_gemm(dev(x), K.F16Weight(dev(w)), bias=dev(b), act=_lib.ACT_GELU_TANH))
    ref = O.gelu((O.matmul(x, w.T) + b).astype(np.float16))
    assert rel_err(got, ref) <= 1e-2


# ---------------------------------------------------------------- FP8 (bit-exact codecs)
@pytest.mark.parametrize("fmt", ["F143", "F152"])
@pytest.mark.parametrize("scale", [0, -1, 3])
def test_fp8_codecs_bit_exact(K, fmt, scale):
    codes = np.arange(256, dtype=np.uint8)
    s = dev(np.array([scale], np.int32))
    got = host(K.fp8_to_half(dev(codes), s, fmt))
    ref = O.f8_decode(codes, fmt, scale, np.float16)
    ok = codes != 0x80
    assert np.array_equal(got[ok].view(np.uint16), ref[ok].view(np.uint16)) and np.isnan(got[0x80])
    rng = np.random.default_rng(31)
    mx = 240.0 if fmt == "F143" else 57344.0
    x = np.concatenate([rng.standard_normal(20000) * 0.05, rng.uniform(-mx, mx, 20000) * 2.0 ** scale,
                        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504, -65504, 6e-8, -6e-8])]).astype(np.float16)
    # every fp16 value near the grid boundaries: all midpoints between adjacent codes
    tab = O.f8_table(fmt)[:128].astype(np.float64) * 2.0 ** scale
    mids = ((tab[:-1] + tab[1:]) / 2)
    x = np.concatenate([x, mids.astype(np.float16), -mids.astype(np.float16), np.nextafter(mids.astype(np.float16), np.float16(np.inf))])
    got = host(K.half_to_fp8(dev(x), s, fmt))
    ref = O.f8_encode(x, fmt, scale)
    assert np.array_equal(got, ref)
    with pytest.raises(ValueError):
        K.half_to_fp8(dev(x), s, "F999")


@pytest.mark.parametrize("M,Kdim,N", [(1, 4096, 512), (8, 512, 4096), (3, 136, 40), (64, 1024, 64)])
@pytest.mark.parametrize("fmt", ["F143", "F152"])
def test_fp8_gemm_both_modes(K, M, Kdim, N, fmt):
    rng = np.random.default_rng(M + Kdim + N)
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    w = (rng.standard_normal((Kdim, N)) * 0.02).astype(np.float32)          # [K, N] as the graph holds it
    scale = -1
    w8 = O.f8_encode(w, fmt, scale)
    w8[0, 0] = 0x7F if fmt == "F143" else 0x5F                              # the saturation code (+max) / a large finite code
    w8[1, 0] = 0x01                                                          # the smallest subnormal
    sd = dev(np.array([scale], np.int32))
    fw = K.F8Weight(dev(w8), sd, fmt, kn=True)
    ws = K.fp8_gemm_workspace(M, Kdim, "cuda")
    got16 = host(K.fp8_gemm(dev(x), fw, ws))
    ref16 = O.fp8_matmul(x, w8, [scale], [scale], fmt, fmt)
    assert rel_err(got16, ref16) <= 1e-2
    x8 = O.f8_encode(x, "F143", scale)
    got8 = host(K.fp8_gemm(dev(x8), fw, ws, x_scale=sd, x_format="F143"))
    ref8 = O.fp8_matmul(x8, w8, [scale], [scale], "F143", fmt)
    assert rel_err(got8, ref8) <= 1e-2
    # same weights given in [N, K] orientation tile identically
    fw2 = K.F8Weight(dev(np.ascontiguousarray(w8.T)), sd, fmt, kn=False)
    assert torch.equal(fw.tiled, fw2.tiled)


@pytest.mark.parametrize("fmt,scale", [("F143", -3), ("F143", 2), ("F152", -1)])
def test_casts_done_by_the_producer_are_bit_identical(K, fmt, scale):
    """The cast of an FP8 Linear's input done where that input is produced - inside the RMSNorm pass, and in
    the epilogue of a Linear or of a SwiGLU pair, for 1, 12 and 40 rows (three GEMM kernels) - gives the bits
    of the separate pta_half_to_fp8_grid pass."""
    rng = np.random.default_rng(77)
    sd = dev(np.array([scale], np.int32))
    for rows in (1, 12, 40):
        x = (rng.standard_normal((rows, 1024)) * 3).astype(np.float16)
        g = rng.uniform(0.5, 1.5, 1024).astype(np.float16)
        fused = K.rmsnorm_fp8_grid(dev(x), dev(g), 1e-5, sd, fmt)
        two = K.half_to_fp8_grid(K.rmsnorm(dev(x), dev(g), 1e-5), sd, fmt)
        assert torch.equal(fused, two)
        assert np.array_equal(host(two), O.f8_decode(O.f8_encode(O.rms_norm(x, g, 1e-5), fmt, scale), fmt, 0, np.float16))
        N = 8192
        (pg, sg), (pu, su) = [(rng.integers(-128, 128, size=(N, 512), dtype=np.int8),
                               rng.uniform(0.005, 0.02, size=(N,)).astype(np.float16)) for _ in range(2)]
        wg, wu = K.W4Weight(dev(pg), dev(sg)), K.W4Weight(dev(pu), dev(su))
        res = dev(rng.standard_normal((rows, N)).astype(np.float16))
        y = torch.empty((rows, N), dtype=torch.float16, device="cuda")
        y2 = torch.empty_like(y)
        K.linear(dev(x), [wg], [y], residual=res, out_grid=(sd, fmt))
        K.linear(dev(x), [wg], [y2], residual=res)
        assert torch.equal(y, K.half_to_fp8_grid(y2, sd, fmt))
        K.linear(dev(x), [wg, wu], [y, y], swiglu=True, out_grid=(sd, fmt))
        K.linear(dev(x), [wg, wu], [y2, y2], swiglu=True)
        assert torch.equal(y, K.half_to_fp8_grid(y2, sd, fmt))
    with pytest.raises(ValueError):
        K.linear(dev(x), [wg, wu], [y, y2], out_grid=(sd, fmt))          # two plain weights: no output cast
    # every fp16 value through the cast of the norm pass (weight 1: x * r with r = 1 exactly needs rows whose
    # mean square is 1; instead the cast is reached through a Linear with an identity weight and no rounding)
    allv = np.arange(65536, dtype=np.uint16).view(np.float16).reshape(64, 1024)
    eye = np.zeros((16, 1024), np.float16)                              # channel c picks feature c
    eye[np.arange(16), np.arange(16)] = 1
    picked = allv.reshape(-1, 16)                                       # 4096 groups of 16 values
    xs = np.zeros((64, 1024), np.float16)
    w16 = K.F16Weight(dev(eye))
    for g0 in range(0, 4096, 64):
        xs[:, :16] = picked[g0:g0 + 64]
        with np.errstate(invalid="ignore"):
            safe = np.where(np.isfinite(xs), xs, 0).astype(np.float16)  # a NaN or inf would spread over the row's sums
        out = torch.empty((64, 16), dtype=torch.float16, device="cuda")
        K.linear(dev(safe), [w16], [out], out_grid=(sd, fmt))
        ref = O.f8_decode(O.f8_encode(safe[:, :16], fmt, scale), fmt, 0, np.float16)
        assert np.array_equal(host(out).view(np.uint16), ref.view(np.uint16)), f"values of group {g0}"


@pytest.mark.parametrize("M,Kdim,N", [(48, 1024, 8192), (24, 1024, 20480), (48, 1024, 20480)])
def test_fp8_gemm_many_rows_wide_outputs(K, M, Kdim, N):
    """FP8 weights at 17..64 rows; 20480 channels: more 64-channel workgroups than compute units (up to 32 rows in
    workgroups of 16 waves and 128 channels)."""
    rng = np.random.default_rng(22 + N // 4096)
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    w8 = O.f8_encode((rng.standard_normal((Kdim, N)) * 0.02).astype(np.float32), "F143", -1)
    fw = K.F8Weight(dev(w8), dev(np.array([-1], np.int32)), "F143", kn=True)
    got = host(K.fp8_gemm(dev(x), fw, K.fp8_gemm_workspace(M, Kdim, "cuda")))
    assert rel_err(got, O.fp8_matmul(x, w8, [-1], [-1], "F143", "F143")) <= 1e-2


@pytest.mark.parametrize("M", [24, 64])
def test_fp8_gemm_few_outputs_split_k(K, M):
    """FP8 weights, more than 16 rows and 4096 output channels (the attention output / MLP down of the FP8 models at
    17..64 rows): with a workspace the features are split across workgroups; against the oracle and against the
    launch without the split (the same sums in another order), bias and a residual that aliases the output."""
    rng = np.random.default_rng(23 + M)
    Kdim, N = 4096, 4096
    x = rng.standard_normal((M, Kdim)).astype(np.float16)
    w8 = O.f8_encode((rng.standard_normal((Kdim, N)) * 0.02).astype(np.float32), "F143", -1)
    fw = K.F8Weight(dev(w8), dev(np.array([-1], np.int32)), "F143", kn=True)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    ws = K.linear_workspace(M, N, "cuda")
    ws.fill_(0xFF)
    y = dev(res.copy())
    K.linear(dev(x), [fw], [y], bias=dev(bias), residual=y, workspace=ws)
    plain = dev(res.copy())
    K.linear(dev(x), [fw], [plain], bias=dev(bias), residual=plain)
    ref = ((O.fp8_matmul(x, w8, [-1], [-1], "F143", "F143") + bias).astype(np.float16) + res).astype(np.float16)
    assert rel_err(host(y), ref) <= 1e-2 and rel_err(host(y), host(plain)) <= 2e-3


def test_fp8_gemm_exact_on_representable_values(K):
    """Small integers and powers of two are exact in F143, in fp16 and in the fp32 sums."""
    rng = np.random.default_rng(32)
    M, Kdim, N = 4, 256, 32
    x = rng.integers(-2, 3, size=(M, Kdim)).astype(np.float16)
    w = rng.choice([-4.0, -1.5, -0.25, 0.0, 0.5, 1.0, 3.0], size=(N, Kdim)).astype(np.float32)
    w8 = O.f8_encode(w, "F143", 0)
    assert np.array_equal(O.f8_decode(w8, "F143", 0, np.float32), w)
    s0 = dev(np.array([0], np.int32))
    got = host(K.fp8_gemm(dev(x), K.F8Weight(dev(w8), s0, "F143"), K.fp8_gemm_workspace(M, Kdim, "cuda")))
    assert np.array_equal(got.astype(np.float64), x.astype(np.float64) @ w.T.astype(np.float64))


# ---------------------------------------------------------------- norms
@pytest.mark.parametrize("rows,cols", [(1, 4096), (16, 4096), (3, 768), (2, 8)])
def test_rmsnorm(K, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float16)
    g = rng.uniform(0.5, 1.5, cols).astype(np.float16)
    got = host(K.rmsnorm(dev(x), dev(g), 1e-5))
    ref = O.rms_norm(x, g, 1e-5)
    # identical up to the rounding of the inverse RMS (summation order): 2 fp16 ulp
    assert np.abs(got.astype(np.float32) - ref.astype(np.float32)).max() <= 2 * 2.0 ** -10 * np.abs(ref).max()
    assert (got.view(np.uint16) == ref.view(np.uint16)).mean() > 0.5


@pytest.mark.parametrize("rows,cols", [(1, 768), (1, 4096), (32, 4096), (5, 1024)])
def test_layer_norm_ce(K, rows, cols):
    rng = np.random.default_rng(rows * 3 + cols)
    x = (rng.standard_normal((rows, cols)) * 2 + 0.3).astype(np.float16)
    g = rng.uniform(0.5, 1.5, cols).astype(np.float16)
    b = rng.standard_normal(cols).astype(np.float16)
    got = host(K.layer_norm_ce(dev(x), dev(g), dev(b), 1e-5))
    ref = O.layer_norm_ce(x, g, b, 1e-5, rows, 1, cols)
    assert np.abs(got.astype(np.float32) - ref.astype(np.float32)).max() <= 4 * 2.0 ** -10 * np.abs(ref).max()


def test_layer_norm_ce_guards(K):
    x = dev(np.zeros((1, 8192), np.float16))
    g = dev(np.ones(8192, np.float16))
    with pytest.raises(ValueError):
        K.layer_norm_ce(x, g, g, 1e-5)
    with pytest.raises(ValueError):
        K.layer_norm_ce(dev(np.zeros((1, 64), np.float32)), g, g, 1e-5)


# ---------------------------------------------------------------- softmax
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("stable", [False, True])
@pytest.mark.parametrize("rows,n", [(1, 128), (32, 2048), (7, 33)])
def test_softmax_ce(K, dtype, stable, rows, n):
    rng = np.random.default_rng(rows + n)
    x = (rng.standard_normal((rows, n)) * 2).astype(dtype)
    x[:, n // 2:] -= 10000          # the attention mask value
    got = host(K.softmax_ce(dev(x), stable))
    ref = O.softmax_ce(x, -1, stable)
    tol = 3e-3 if dtype == np.float16 else 1e-5
    assert np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() <= tol
    assert np.all(got[:, n // 2:] == 0)


# ---------------------------------------------------------------- KV cache (bit-exact)
@pytest.mark.parametrize("shape,axis,max_len,dtype", [((2, 1, 3, 1, 8), 3, 5, np.float16), ((2, 2, 4, 1, 128), 3, 7, np.float16),
                                                      ((3, 1, 5), 1, 4, np.float32), ((2, 1, 2, 1, 3), 3, 6, np.float16)])
def test_kv_cache_ring_matches_shift_register(K, shape, axis, max_len, dtype):
    rng = np.random.default_rng(17)
    ref_op = O.KVCache(max_len, axis, 1)
    outer = int(np.prod(shape[:axis]))
    inner = int(np.prod(shape[axis + 1:]))
    out_shape = list(shape)
    out_shape[axis] = max_len
    ring = torch.empty((outer, max_len, inner), dtype=torch.from_numpy(np.zeros(1, dtype)).dtype, device="cuda")
    ring.fill_(7)                                            # stale contents must never show
    cache_lit = torch.full(out_shape, 7, dtype=ring.dtype, device="cuda")
    clone = torch.empty_like(cache_lit)
    view = torch.empty(out_shape, dtype=ring.dtype, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    for it in range(max_len + 3):
        upd = rng.standard_normal(shape).astype(dtype)
        ref = ref_op(it, upd)
        step.fill_(it)
        u = dev(upd)
        K.kv_cache_append(ring, u, step, outer, max_len, inner)
        K.kv_cache_read(ring, view, step, outer, max_len, inner)
        K.kv_cache_update(cache_lit, clone, u, step, axis)
        assert np.array_equal(host(view), ref), f"ring view differs at step {it}"
        assert np.array_equal(host(cache_lit), ref), f"literal cache differs at step {it}"
    # step 0 again zeroes the history
    upd = rng.standard_normal(shape).astype(dtype)
    ref = ref_op(0, upd)
    step.fill_(0)
    K.kv_cache_append(ring, dev(upd), step, outer, max_len, inner)
    K.kv_cache_read(ring, view, step, outer, max_len, inner)
    assert np.array_equal(host(view), ref)


def test_kv_cache_pipeline(K):
    rng = np.random.default_rng(23)
    max_len, max_bps, shape = 4, 3, (2, 2, 1, 16)
    ref_op = O.KVCachePipeline(max_len, max_bps)
    outer, inner = 4, 16
    ring = torch.full((max_bps, outer, max_len, inner), 5, dtype=torch.float16, device="cuda")
    view = torch.empty((2, 2, max_len, 16), dtype=torch.float16, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    for it in range(max_bps * (max_len + 2)):
        upd = rng.standard_normal(shape).astype(np.float16)
        ref = ref_op(it, upd)
        step.fill_(it)
        K.kv_cache_append(ring, dev(upd), step, outer, max_len, inner, max_bps)
        K.kv_cache_read(ring, view, step, outer, max_len, inner, max_bps)
        assert np.array_equal(host(view), ref), f"pipeline cache differs at step {it}"


# ---------------------------------------------------------------- attention
def _attention_reference(family, qs, ks, vs, max_len, D, fp8_cache=False):
    """Runs the oracle chain step by step; returns the context vectors per step."""
    B, Hq = qs[0].shape[0], qs[0].shape[1]
    Hkv = ks[0].shape[1]
    cache = O.KVCache(max_len, 3, 1, fp8=fp8_cache)
    mask = np.full((B, max_len), -10000, np.float16)
    mask[:, 0] = 0
    outs = []
    for step, (q, k, v) in enumerate(zip(qs, ks, vs)):
        q4 = q.reshape(B, Hq, 1, D)
        k4 = k.reshape(B, Hkv, 1, D)
        v4 = v.reshape(B, Hkv, 1, D)
        if family == "llama":
            sin, cos = O.llama_sincos(step, D)
            q4, k4 = O.llama_rope(q4, sin, cos), O.llama_rope(k4, sin, cos)
        elif family == "glm2":
            cos, sin = O.glm2_sincos(step, D)
            q4 = np.swapaxes(O.glm2_rope(np.swapaxes(q4, 1, 2), cos, sin), 1, 2)
            k4 = np.swapaxes(O.glm2_rope(np.swapaxes(k4, 1, 2), cos, sin), 1, 2)
        past = cache(step, np.stack([k4, v4]))
        kk, vv = past[0], past[1]
        if Hkv != Hq:
            kk = np.repeat(kk, Hq // Hkv, axis=1)
            vv = np.repeat(vv, Hq // Hkv, axis=1)
        scale = None if family == "gpt2" else 1 / np.sqrt(D)
        sdt = np.float32 if family == "llama" else np.float16
        ctx = O.attention_scores_to_context(q4, np.swapaxes(kk, 2, 3), vv, mask[:, None, None, :], scale, sdt)
        outs.append(np.swapaxes(ctx, 1, 2).reshape(B, Hq * D))
        if step + 1 < max_len:
            mask[:, step + 1] = 0
    return outs


@pytest.mark.parametrize("family,B,Hq,Hkv,D,max_len,steps", [("llama", 2, 4, 4, 128, 100, 70), ("gpt2", 1, 12, 12, 64, 40, 40),
                                                             ("glm2", 2, 8, 2, 128, 150, 80), ("llama", 1, 2, 2, 128, 16, 20),
                                                             # rings of more than 256 rows: several chunks per head and the merging launch
                                                             ("llama", 2, 4, 4, 128, 300, 330), ("gpt2", 1, 12, 12, 64, 320, 100),
                                                             # sixteen query heads per KV head: the grouped kernel on the
                                                             # matrix unit (one chunk and several, a ring that wraps)
                                                             ("glm2", 2, 32, 2, 128, 150, 170), ("llama", 1, 16, 1, 64, 40, 50),
                                                             ("glm2", 2, 16, 1, 64, 300, 200),
                                                             # 128 (sequence, KV head) pairs: one chunk each, several steps per wave
                                                             ("glm2", 64, 32, 2, 64, 200, 170)])
def test_rope_append_attention(K, family, B, Hq, Hkv, D, max_len, steps):
    from poptransformer_amd import _lib
    rng = np.random.default_rng(B + Hq + D)
    qs = [(rng.standard_normal((B, Hq, D)) * (0.3 if family == "gpt2" else 1.0)).astype(np.float16) for _ in range(steps)]
    ks = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(steps)]
    vs = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(steps)]
    refs = _attention_reference(family, qs, ks, vs, max_len, D)   # steps > max_len drops the oldest rows
    rope = {"llama": _lib.ROPE_LLAMA, "glm2": _lib.ROPE_GLM2, "gpt2": _lib.ROPE_NONE}[family]
    inv = None
    if family == "llama":
        inv = dev(np.array([1.0 / (10000 ** (i / D)) for i in range(0, D, 2)]).astype(np.float16))
    elif family == "glm2":
        inv = dev(np.array([1.0 / (10000 ** (i / (D // 2))) for i in range(0, D // 2, 2)]).astype(np.float32))
    ring = torch.full((2 * B * Hkv, max_len, D), float("nan"), dtype=torch.float16, device="cuda")
    ws = K.decode_attention_workspace(B, Hq, D, max_len, "cuda")
    q_rot = torch.empty((B, Hq, D), dtype=torch.float16, device="cuda")
    out = torch.empty((B, Hq * D), dtype=torch.float16, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    for it in range(steps):
        step.fill_(it)
        K.qkv_rope_append(dev(qs[it]), dev(ks[it]), dev(vs[it]), q_rot, ring, step, inv, B, Hq, Hkv, D, max_len, rope)
        K.decode_attention(q_rot, ring, step, ws, out, B, Hq, Hkv, D, max_len, family != "gpt2")
        got = host(out)
        assert np.isfinite(got).all(), f"non-finite output at step {it}"
        assert rel_err(got, refs[it]) <= 1e-2, f"step {it}"


@pytest.mark.parametrize("family,B,Hq,Hkv,D,max_len,steps", [("llama", 2, 4, 4, 128, 100, 130), ("gpt2", 1, 12, 12, 64, 40, 45),
                                                             ("glm2", 3, 8, 2, 128, 150, 90), ("glm2", 3, 8, 2, 128, 320, 350),
                                                             ("glm2", 2, 32, 2, 128, 150, 170), ("llama", 1, 16, 1, 64, 70, 90),
                                                             ("glm2", 64, 32, 2, 64, 200, 170)])
def test_attention_with_its_own_preparation_is_bit_identical(K, family, B, Hq, Hkv, D, max_len, steps):
    """pta_decode_attention_qkv (rotary + append inside the attention pass) against the two separate calls: the
    same context vectors and the same ring, bit for bit, at every step including those after the ring has
    wrapped, with grouped KV heads and with strided q | k | v rows."""
    from poptransformer_amd import _lib
    rng = np.random.default_rng(B * 5 + Hq + D)
    rope = {"llama": _lib.ROPE_LLAMA, "glm2": _lib.ROPE_GLM2, "gpt2": _lib.ROPE_NONE}[family]
    inv = None
    if family == "llama":
        inv = dev(np.array([1.0 / (10000 ** (i / D)) for i in range(0, D, 2)]).astype(np.float16))
    elif family == "glm2":
        inv = dev(np.array([1.0 / (10000 ** (i / (D // 2))) for i in range(0, D // 2, 2)]).astype(np.float32))
    row = (Hq + 2 * Hkv) * D
    rings = [torch.zeros((2 * B * Hkv, max_len, D), dtype=torch.float16, device="cuda") for _ in range(2)]
    wss = [K.decode_attention_workspace(B, Hq, D, max_len, "cuda") for _ in range(2)]
    q_rot = torch.empty((B, Hq, D), dtype=torch.float16, device="cuda")
    outs = [torch.empty((B, Hq * D), dtype=torch.float16, device="cuda") for _ in range(2)]
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    for it in range(steps):
        qkv = dev(rng.standard_normal((B, row)).astype(np.float16))          # one row holds q | k | v
        q, k, v = qkv, qkv[:, Hq * D:], qkv[:, (Hq + Hkv) * D:]
        step.fill_(it)
        K.qkv_rope_append(q, k, v, q_rot, rings[0], step, inv, B, Hq, Hkv, D, max_len, rope, row, row, row)
        K.decode_attention(q_rot, rings[0], step, wss[0], outs[0], B, Hq, Hkv, D, max_len, family != "gpt2")
        K.decode_attention_qkv(q, k, v, rings[1], step, inv, wss[1], outs[1], B, Hq, Hkv, D, max_len, rope,
                               family != "gpt2", row, row, row)
        assert torch.equal(outs[0], outs[1]), f"context differs at step {it}"
    assert torch.equal(rings[0], rings[1])
    # the same pass leaving its context vectors on an FP8 grid: the bits of the separate cast (the ring already holds
    # this step's row: the append writes the same values again)
    for fmt, scale in (("F143", -1), ("F152", 2)):
        sd = dev(np.array([scale], np.int32))
        on_grid = torch.empty_like(outs[1])
        K.decode_attention_qkv(q, k, v, rings[1], step, inv, wss[1], on_grid, B, Hq, Hkv, D, max_len, rope,
                               family != "gpt2", row, row, row, out_grid=(sd, fmt))
        assert torch.equal(on_grid, K.half_to_fp8_grid(outs[1], sd, fmt))
    assert torch.equal(rings[0], rings[1])


@pytest.mark.parametrize("family,B,Hq,Hkv,D,max_len,first,rows", [("llama", 2, 4, 4, 128, 160, 0, 32), ("llama", 1, 4, 4, 128, 160, 70, 64),
                                                                  ("gpt2", 3, 4, 4, 64, 64, 5, 21), ("glm2", 2, 8, 2, 128, 200, 64, 17),
                                                                  ("llama", 1, 4, 4, 128, 300, 3, 200), ("glm2", 2, 8, 2, 128, 256, 30, 130),
                                                                  ("llama", 2, 2, 2, 128, 64, 0, 15), ("llama", 1, 2, 2, 128, 64, 0, 16),
                                                                  ("glm2", 2, 8, 2, 64, 96, 10, 40), ("gpt2", 1, 6, 6, 64, 200, 20, 150)])
def test_prompt_rows_equal_the_loop(K, family, B, Hq, Hkv, D, max_len, first, rows):
    """pta_prompt_rope_append + pta_prompt_attention over `rows` positions at once against the oracle's
    position-by-position attention (1e-2) and against the per-position calls: the ring is bit-identical, the
    context vectors agree to rounding (the split of the cache rows over workgroups differs)."""
    from poptransformer_amd import _lib
    rng = np.random.default_rng(B + rows + D)
    steps = first + rows
    qs = [(rng.standard_normal((B, Hq, D)) * (0.3 if family == "gpt2" else 1.0)).astype(np.float16) for _ in range(steps)]
    ks = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(steps)]
    vs = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(steps)]
    refs = _attention_reference(family, qs, ks, vs, max_len, D)
    rope = {"llama": _lib.ROPE_LLAMA, "glm2": _lib.ROPE_GLM2, "gpt2": _lib.ROPE_NONE}[family]
    inv = None
    if family == "llama":
        inv = dev(np.array([1.0 / (10000 ** (i / D)) for i in range(0, D, 2)]).astype(np.float16))
    elif family == "glm2":
        inv = dev(np.array([1.0 / (10000 ** (i / (D // 2))) for i in range(0, D // 2, 2)]).astype(np.float32))
    rings = [torch.zeros((2 * B * Hkv, max_len, D), dtype=torch.float16, device="cuda") for _ in range(2)]
    ws = K.decode_attention_workspace(B, Hq, D, max_len, "cuda")
    q_rot = torch.empty((B, Hq, D), dtype=torch.float16, device="cuda")
    out = torch.empty((B, Hq * D), dtype=torch.float16, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    loop_out = []
    for it in range(steps):                       # ring 0: the loop, one position per call
        step.fill_(it)
        K.qkv_rope_append(dev(qs[it]), dev(ks[it]), dev(vs[it]), q_rot, rings[0], step, inv, B, Hq, Hkv, D, max_len, rope)
        K.decode_attention(q_rot, rings[0], step, ws, out, B, Hq, Hkv, D, max_len, family != "gpt2")
        loop_out.append(host(out))
        if it < first:                            # ring 1 receives the positions before the pass the same way
            K.qkv_rope_append(dev(qs[it]), dev(ks[it]), dev(vs[it]), q_rot, rings[1], step, inv, B, Hq, Hkv, D, max_len, rope)
    # rows of the pass: sequence-major, then position
    stack = lambda xs: dev(np.stack(xs[first:], axis=1).reshape(B * rows, -1))
    q_rows = torch.empty((B * rows, Hq, D), dtype=torch.float16, device="cuda")
    out_rows = torch.empty((B * rows, Hq * D), dtype=torch.float16, device="cuda")
    ws_rows = K.decode_attention_workspace(B * rows, Hq, D, max_len, "cuda")
    step.fill_(first)
    K.prompt_rope_append(stack(qs), stack(ks), stack(vs), q_rows, rings[1], step, inv, B, rows, Hq, Hkv, D, max_len, rope)
    K.prompt_attention(q_rows, rings[1], step, ws_rows, out_rows, B, rows, Hq, Hkv, D, max_len, family != "gpt2")
    assert torch.equal(rings[0], rings[1])
    got = host(out_rows).reshape(B, rows, Hq * D)
    for r in range(rows):
        assert rel_err(got[:, r], refs[first + r]) <= 1e-2, f"row {r} against the oracle"
        assert rel_err(got[:, r], loop_out[first + r]) <= 2e-3, f"row {r} against the loop"
    with pytest.raises(ValueError):
        K.prompt_attention(q_rows, rings[1], step, ws, out_rows, B, rows, Hq, Hkv, D, max_len, True)   # workspace of one row


def _prefix_reference(family, qs, ks, vs, D, rows, fp8_cache=False):
    """The oracle's attention chain for the positions in `rows`, each over the cache rows 0..r it sees (newest first,
    as the KVCache op holds them) instead of over a cache that is stepped through every position: a masked row's
    probability is exactly zero in both chains, so the two differ only in the order of sums
    (test_prefix_reference_is_the_stepped_reference).  Returns {r: context [B, Hq * D]}."""
    B, Hq, Hkv = qs[0].shape[0], qs[0].shape[1], ks[0].shape[1]

    def rotated(x, pos):
        x4 = x.reshape(B, -1, 1, D)
        if family == "llama":
            sin, cos = O.llama_sincos(pos, D)
            return O.llama_rope(x4, sin, cos)
        if family == "glm2":
            cos, sin = O.glm2_sincos(pos, D)
            return np.swapaxes(O.glm2_rope(np.swapaxes(x4, 1, 2), cos, sin), 1, 2)
        return x4

    def stored(x4):
        return O.f8_decode(O.f8_encode(x4, "F143", O.KVCache.FP8_SCALE), "F143", O.KVCache.FP8_SCALE, np.float16) if fp8_cache else x4

    last = max(rows)
    kc = [stored(rotated(ks[p], p)) for p in range(last + 1)]
    vc = [stored(vs[p].reshape(B, Hkv, 1, D)) for p in range(last + 1)]
    scale = None if family == "gpt2" else 1 / np.sqrt(D)
    sdt = np.float32 if family == "llama" else np.float16
    out = {}
    for r in rows:
        kk = np.concatenate(kc[r::-1], axis=2)
        vv = np.concatenate(vc[r::-1], axis=2)
        if Hkv != Hq:
            kk, vv = np.repeat(kk, Hq // Hkv, axis=1), np.repeat(vv, Hq // Hkv, axis=1)
        ctx = O.attention_scores_to_context(rotated(qs[r], r), np.swapaxes(kk, 2, 3), vv, np.zeros((B, 1, 1, r + 1), np.float16), scale, sdt)
        out[r] = np.swapaxes(ctx, 1, 2).reshape(B, Hq * D)
    return out


@pytest.mark.parametrize("family,fp8", [("llama", False), ("glm2", False), ("gpt2", False), ("llama", True)])
def test_prefix_reference_is_the_stepped_reference(family, fp8):
    """CPU only: _prefix_reference against _attention_reference (the oracle stepped through every position)."""
    rng = np.random.default_rng(5)
    B, Hq, Hkv, D, n = 2, 4, 2 if family == "glm2" else 4, 64, 40
    qs = [(rng.standard_normal((B, Hq, D)) * (0.3 if family == "gpt2" else 1.0)).astype(np.float16) for _ in range(n)]
    ks = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(n)]
    vs = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(n)]
    stepped = _attention_reference(family, qs, ks, vs, 48, D, fp8_cache=fp8)
    for r, ctx in _prefix_reference(family, qs, ks, vs, D, [0, 1, 17, 39], fp8_cache=fp8).items():
        assert rel_err(ctx, stepped[r]) <= 2e-3, f"position {r}"


@pytest.mark.parametrize("D,kv8", [(64, False), (128, False), (64, True), (128, True)])
def test_prompt_attention_two_row_groups(K, D, kv8):
    """A pass with enough (sequence, head, 128 rows) tiles to fill every compute unit twice takes the workgroups of
    128 rows whose waves hold two row groups each: 4 sequences x 32 heads x 512 rows, fp16 and F143 rings, head sizes
    64 and 128, against the oracle's chain at rows spread over the pass (first and last rows of row groups, of
    128-row tiles and of the 32-row stages of cache rows)."""
    from poptransformer_amd import _lib
    B, Hq, Hkv, rows, max_len = 4, 32, 32, 512, 520
    print(f"case: prompt attention, two row groups per wave, head size {D}, {'F143' if kv8 else 'fp16'} ring", flush=True)
    rng = np.random.default_rng(D + kv8)
    qs = [rng.standard_normal((B, Hq, D)).astype(np.float16) for _ in range(rows)]
    ks = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(rows)]
    vs = [(rng.standard_normal((B, Hkv, D)) * (40.0 if kv8 else 1.0)).astype(np.float16) for _ in range(rows)]
    check = [0, 1, 15, 16, 31, 32, 33, 63, 64, 127, 128, 129, 200, 255, 256, 300, 383, 384, 447, 480, 510, 511]
    refs = _prefix_reference("llama", qs, ks, vs, D, check, fp8_cache=kv8)
    inv = dev(np.array([1.0 / (10000 ** (i / D)) for i in range(0, D, 2)]).astype(np.float16))
    ring = torch.zeros((2 * B * Hkv, max_len, D), dtype=torch.uint8 if kv8 else torch.float16, device="cuda")
    stack = lambda xs: dev(np.stack(xs, axis=1).reshape(B * rows, -1))
    q_rows = torch.empty((B * rows, Hq, D), dtype=torch.float16, device="cuda")
    out_rows = torch.empty((B * rows, Hq * D), dtype=torch.float16, device="cuda")
    ws_rows = K.decode_attention_workspace(B * rows, Hq, D, max_len, "cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    kw = dict(kv_scale=1) if kv8 else {}
    K.prompt_rope_append(stack(qs), stack(ks), stack(vs), q_rows, ring, step, inv, B, rows, Hq, Hkv, D, max_len, _lib.ROPE_LLAMA, **kw)
    K.prompt_attention(q_rows, ring, step, ws_rows, out_rows, B, rows, Hq, Hkv, D, max_len, True, **kw)
    got = host(out_rows).reshape(B, rows, Hq * D)
    assert np.isfinite(got).all()
    for r in check:
        assert rel_err(got[:, r], refs[r]) <= 1e-2, f"row {r}"


def test_decode_attention_beyond_1024_rows_grouped_heads(K):
    """The ChatGLM2 benchmark's attention shape: 8 sequences, 32 query heads on 2 KV heads of 128, a ring of 4096,
    contexts 1100..1103 (the splits of a (sequence, head) all hold rows).  The ring is filled by passes of 256
    positions, the next positions run one per call through the pass that prepares its own operands and through the two
    separate calls."""
    from poptransformer_amd import _lib
    B, Hq, Hkv, D, max_len, n0, more = 8, 32, 2, 128, 4096, 1100, 4
    print("case: decode attention at context 1100, 32 query / 2 KV heads, ring of 4096", flush=True)
    rng = np.random.default_rng(11)
    n = n0 + more
    qs = [rng.standard_normal((B, Hq, D)).astype(np.float16) for _ in range(n)]
    ks = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(n)]
    vs = [rng.standard_normal((B, Hkv, D)).astype(np.float16) for _ in range(n)]
    refs = _prefix_reference("glm2", qs, ks, vs, D, list(range(n0, n)))
    inv = dev(np.array([1.0 / (10000 ** (i / (D // 2))) for i in range(0, D // 2, 2)]).astype(np.float32))
    rings = [torch.zeros((2 * B * Hkv, max_len, D), dtype=torch.float16, device="cuda") for _ in range(2)]
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    R = 256
    for p0 in range(0, n0, R):
        rc = min(R, n0 - p0)
        stack = lambda xs: dev(np.stack(xs[p0:p0 + rc], axis=1).reshape(B * rc, -1))
        q_rows = torch.empty((B * rc, Hq, D), dtype=torch.float16, device="cuda")
        step.fill_(p0)
        for ring in rings:
            K.prompt_rope_append(stack(qs), stack(ks), stack(vs), q_rows, ring, step, inv, B, rc, Hq, Hkv, D, max_len, _lib.ROPE_GLM2)
    ws = K.decode_attention_workspace(B, Hq, D, max_len, "cuda")
    q_rot = torch.empty((B, Hq, D), dtype=torch.float16, device="cuda")
    outs = [torch.empty((B, Hq * D), dtype=torch.float16, device="cuda") for _ in range(2)]
    for it in range(n0, n):
        step.fill_(it)
        q, k, v = dev(qs[it]), dev(ks[it]), dev(vs[it])
        K.qkv_rope_append(q, k, v, q_rot, rings[0], step, inv, B, Hq, Hkv, D, max_len, _lib.ROPE_GLM2)
        K.decode_attention(q_rot, rings[0], step, ws, outs[0], B, Hq, Hkv, D, max_len, True)
        K.decode_attention_qkv(q, k, v, rings[1], step, inv, ws, outs[1], B, Hq, Hkv, D, max_len, _lib.ROPE_GLM2, True)
        assert rel_err(host(outs[0]), refs[it]) <= 1e-2, f"context {it}"
        assert torch.equal(outs[0], outs[1]), f"context {it}: the pass that prepares its operands differs"
    assert torch.equal(rings[0], rings[1])


@pytest.mark.parametrize("family,B,Hq,Hkv,D,max_len,steps", [("llama", 2, 4, 4, 128, 100, 130), ("glm2", 2, 8, 2, 128, 96, 70),
                                                             ("gpt2", 1, 4, 4, 64, 48, 50)])
def test_fp8_kv_cache_attention(K, family, B, Hq, Hkv, D, max_len, steps):
    """KV rings of F143 bytes (metadata scale 1): the stored bytes are bit-exact against the oracle's cast of the
    rotated keys and the values, the context vectors within 1e-2 of the oracle's attention over the cast-back
    cache, at every step including those after the ring has wrapped; the pass that prepares its own operands
    (pta_decode_attention_qkv_f8) gives the same bytes and the same context, bit for bit, as the two calls; and
    several positions at once (rows > 1) leave the same bytes as the loop."""
    from poptransformer_amd import _lib
    rng = np.random.default_rng(B + Hq + D + 1)
    qs = [(rng.standard_normal((B, Hq, D)) * (0.3 if family == "gpt2" else 1.0)).astype(np.float16) for _ in range(steps)]
    # GPT-2's chain has no 1/sqrt(D) and an fp16 softmax without max subtraction: keep its scores small
    ks = [(rng.standard_normal((B, Hkv, D)) * (1.0 if family == "gpt2" else 2.0)).astype(np.float16) for _ in range(steps)]
    vs = [(rng.standard_normal((B, Hkv, D)) * 150.0).astype(np.float16) for _ in range(steps)]     # some values saturate at 480
    refs = _attention_reference(family, qs, ks, vs, max_len, D, fp8_cache=True)
    rope = {"llama": _lib.ROPE_LLAMA, "glm2": _lib.ROPE_GLM2, "gpt2": _lib.ROPE_NONE}[family]
    inv = None
    if family == "llama":
        inv = dev(np.array([1.0 / (10000 ** (i / D)) for i in range(0, D, 2)]).astype(np.float16))
    elif family == "glm2":
        inv = dev(np.array([1.0 / (10000 ** (i / (D // 2))) for i in range(0, D // 2, 2)]).astype(np.float32))
    rings = [torch.zeros((2 * B * Hkv, max_len, D), dtype=torch.uint8, device="cuda") for _ in range(3)]
    ws = K.decode_attention_workspace(B, Hq, D, max_len, "cuda")
    q_rot = torch.empty((B, Hq, D), dtype=torch.float16, device="cuda")
    outs = [torch.empty((B, Hq * D), dtype=torch.float16, device="cuda") for _ in range(2)]
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    for it in range(steps):
        step.fill_(it)
        q, k, v = dev(qs[it]), dev(ks[it]), dev(vs[it])
        K.prompt_rope_append(q, k, v, q_rot, rings[0], step, inv, B, 1, Hq, Hkv, D, max_len, rope, kv_scale=1)
        K.prompt_attention(q_rot, rings[0], step, ws, outs[0], B, 1, Hq, Hkv, D, max_len, family != "gpt2", kv_scale=1)
        K.decode_attention_qkv(q, k, v, rings[1], step, inv, ws, outs[1], B, Hq, Hkv, D, max_len, rope, family != "gpt2",
                               kv_scale=1)
        got = host(outs[0])
        assert np.isfinite(got).all()
        assert rel_err(got, refs[it]) <= 1e-2, f"step {it}"
        assert torch.equal(outs[0], outs[1]), f"step {it}: the fused pass differs"
    assert torch.equal(rings[0], rings[1])
    # the bytes of the last max_len positions against the oracle's cast (position p sits in ring row p % max_len)
    ring = host(rings[0]).reshape(2, B, Hkv, max_len, D)
    for p_ in range(max(0, steps - max_len), steps):
        k4 = ks[p_].reshape(B, Hkv, 1, D)
        if family == "llama":
            sin, cos = O.llama_sincos(p_, D)
            k4 = O.llama_rope(k4, sin, cos)
        elif family == "glm2":
            cos, sin = O.glm2_sincos(p_, D)
            k4 = np.swapaxes(O.glm2_rope(np.swapaxes(k4, 1, 2), cos, sin), 1, 2)
        assert np.array_equal(ring[0, :, :, p_ % max_len], O.f8_encode(k4[:, :, 0], "F143", 1)), f"key bytes of position {p_}"
        assert np.array_equal(ring[1, :, :, p_ % max_len], O.f8_encode(vs[p_], "F143", 1)), f"value bytes of position {p_}"
    # the first `rows` positions at once
    rows = min(32, max_len)
    stack = lambda xs: dev(np.stack(xs[:rows], axis=1).reshape(B * rows, -1))
    q_rows = torch.empty((B * rows, Hq, D), dtype=torch.float16, device="cuda")
    out_rows = torch.empty((B * rows, Hq * D), dtype=torch.float16, device="cuda")
    ws_rows = K.decode_attention_workspace(B * rows, Hq, D, max_len, "cuda")
    step.fill_(0)
    K.prompt_rope_append(stack(qs), stack(ks), stack(vs), q_rows, rings[2], step, inv, B, rows, Hq, Hkv, D, max_len, rope, kv_scale=1)
    K.prompt_attention(q_rows, rings[2], step, ws_rows, out_rows, B, rows, Hq, Hkv, D, max_len, family != "gpt2", kv_scale=1)
    got = host(out_rows).reshape(B, rows, Hq * D)
    for r in range(rows):
        assert rel_err(got[:, r], refs[r]) <= 1e-2, f"row {r}"
    more = min(40, steps - rows)
    if max_len >= rows + more and more >= 16:
        # and the next `more` (on the matrix unit, the cache rows staged 32 at a time, the last step ragged)
        stack2 = lambda xs: dev(np.stack(xs[rows:rows + more], axis=1).reshape(B * more, -1))
        q2 = torch.empty((B * more, Hq, D), dtype=torch.float16, device="cuda")
        out2 = torch.empty((B * more, Hq * D), dtype=torch.float16, device="cuda")
        ws2 = K.decode_attention_workspace(B * more, Hq, D, max_len, "cuda")
        step.fill_(rows)
        K.prompt_rope_append(stack2(qs), stack2(ks), stack2(vs), q2, rings[2], step, inv, B, more, Hq, Hkv, D, max_len, rope, kv_scale=1)
        K.prompt_attention(q2, rings[2], step, ws2, out2, B, more, Hq, Hkv, D, max_len, family != "gpt2", kv_scale=1)
        got2 = host(out2).reshape(B, more, Hq * D)
        for r in range(more):
            assert rel_err(got2[:, r], refs[rows + r]) <= 1e-2, f"row {rows + r}"
        assert torch.equal(rings[2][:, :rows + more], rings[0][:, :rows + more]) or steps > max_len      # the loop's ring has wrapped by then
    with pytest.raises(ValueError):
        K.prompt_attention(q_rows, rings[2].view(torch.float16), step, ws_rows, out_rows, B, rows, Hq, Hkv, D, max_len, True, kv_scale=1)


def test_rope_bit_exact(K):
    """q after rotary embedding and the appended key row are pure fp16 elementwise work: bit-exact."""
    from poptransformer_amd import _lib
    rng = np.random.default_rng(2)
    B, H, D, max_len = 2, 3, 128, 64
    inv = dev(np.array([1.0 / (10000 ** (i / D)) for i in range(0, D, 2)]).astype(np.float16))
    ring = torch.zeros((2 * B * H, max_len, D), dtype=torch.float16, device="cuda")
    q_rot = torch.empty((B, H, D), dtype=torch.float16, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    for it in (0, 1, 5, 37, 63):
        q = rng.standard_normal((B, H, D)).astype(np.float16)
        k = rng.standard_normal((B, H, D)).astype(np.float16)
        v = rng.standard_normal((B, H, D)).astype(np.float16)
        step.fill_(it)
        K.qkv_rope_append(dev(q), dev(k), dev(v), q_rot, ring, step, inv, B, H, H, D, max_len, _lib.ROPE_LLAMA)
        sin, cos = O.llama_sincos(it, D)
        qr = O.llama_rope(q.reshape(B, H, 1, D), sin, cos).reshape(B, H, D)
        kr = O.llama_rope(k.reshape(B, H, 1, D), sin, cos).reshape(B, H, D)
        r = host(ring).reshape(2, B, H, max_len, D)
        # sin/cos of the same fp16 angle may differ by one fp16 ulp between libm and the device
        assert np.abs(host(q_rot).astype(np.float32) - qr.astype(np.float32)).max() <= 2 ** -9 * 4
        assert np.abs(r[0, :, :, it].astype(np.float32) - kr.astype(np.float32)).max() <= 2 ** -9 * 4
        assert np.array_equal(r[1, :, :, it], v)


# ---------------------------------------------------------------- RWKV pieces
def _lib_act(name):
    from poptransformer_amd import _lib
    return {"none": _lib.ACT_NONE, "sigmoid": _lib.ACT_SIGMOID, "relu_square": _lib.ACT_RELU_SQUARE}[name]


@pytest.mark.parametrize("B,d,N", [(1, 4096, 4096), (3, 256, 512), (4, 1024, 2048)])
@pytest.mark.parametrize("with_norm", [True, False])
def test_token_shift_inside_the_linears(K, B, d, N, with_norm):
    """LayerNorm and the RWKV token shift done where the Linears stage their rows (pta_fusion.mix_state): three
    Linears with a mixing vector each, over three consecutive steps of the step counter - against the separate
    launches (layer_norm_ce, rwkv_mix, linear).  The state's two copies take turns: each step reads the rows the
    previous step left and leaves its own; a Linear without a mixing vector in the same launch gets the rows
    unshifted."""
    rng = np.random.default_rng(B + d)
    packed = [rng.integers(-128, 128, size=(N, d // 2), dtype=np.int8) for _ in range(3)]
    scales = [rng.uniform(0.005, 0.02, N).astype(np.float16) for _ in range(3)]
    ws = [K.W4Weight(dev(p_), dev(s_)) for p_, s_ in zip(packed, scales)]
    mixes = [dev(rng.uniform(0, 1, d).astype(np.float16)) for _ in range(2)] + [None]
    g, b = dev(rng.uniform(0.5, 1.5, d).astype(np.float16)), dev((rng.standard_normal(d) * 0.1).astype(np.float16))
    state = torch.zeros((2, B, d), dtype=torch.float16, device="cuda")
    prev = torch.zeros((B, d), dtype=torch.float16, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    for t in range(3):
        x = dev(rng.standard_normal((B, d)).astype(np.float16))
        outs = [torch.empty((B, N), dtype=torch.float16, device="cuda") for _ in range(3)]
        K.linear(x, ws, outs, norm=K.Norm(g, b, 1e-5) if with_norm else None, mixes=mixes, mix=(state, step),
                 acts=[_lib_act("none"), _lib_act("sigmoid"), _lib_act("none")])
        xn = K.layer_norm_ce(x, g, b, 1e-5) if with_norm else x.clone()
        shifted = [torch.empty_like(xn) for _ in range(2)]
        K.rwkv_mix(xn, prev, mixes[:2], shifted)                      # (overwrites prev with xn)
        ref = [torch.empty((B, N), dtype=torch.float16, device="cuda") for _ in range(3)]
        K.linear(None, ws, ref, xs=shifted + [xn], acts=[_lib_act("none"), _lib_act("sigmoid"), _lib_act("none")])
        for o, r_ in zip(outs, ref):
            assert rel_err(host(o), host(r_)) <= (2e-3 if with_norm else 0.0)
        # the rows this step left for the next: the other copy
        left = state[(t + 1) & 1]
        assert rel_err(host(left), host(xn)) <= (2e-3 if with_norm else 0.0)
        step += 1
    with pytest.raises(Exception, match="mix_state"):
        K.linear(dev(np.zeros((8, d), np.float16)), ws, [torch.empty((8, N), dtype=torch.float16, device="cuda") for _ in range(3)],
                 mixes=mixes, mix=(torch.zeros((2, 8, d), dtype=torch.float16, device="cuda"), step))


@pytest.mark.parametrize("rows,cols,nmix", [(1, 768, 3), (5, 4096, 3), (32, 4096, 2), (7, 1000, 1)])
def test_layer_norm_and_token_shift_in_one_launch(K, rows, cols, nmix):
    """pta_layer_norm_ce_mix against pta_layer_norm_ce followed by pta_rwkv_mix, bit for bit (outputs, the state it
    leaves, the normalised rows), and against the oracle's gate of the oracle's LayerNorm."""
    print(f"case: layer norm + token shift, rows {rows}, cols {cols}, {nmix} mixing vectors", flush=True)
    rng = np.random.default_rng(rows * 31 + cols)
    x = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(np.float16)
    prev = rng.standard_normal((rows, cols)).astype(np.float16)
    g = rng.uniform(0.5, 1.5, cols).astype(np.float16)
    b = rng.uniform(-0.5, 0.5, cols).astype(np.float16)
    ws = [rng.uniform(0, 1, cols).astype(np.float16) for _ in range(nmix)]
    wd = [dev(w) for w in ws]
    h = K.layer_norm_ce(dev(x), dev(g), dev(b), 1e-5)
    p_two = dev(prev)
    two = [torch.empty((rows, cols), dtype=torch.float16, device="cuda") for _ in range(nmix)]
    K.rwkv_mix(h, p_two, wd, two)
    p_one = dev(prev)
    one = [torch.empty((rows, cols), dtype=torch.float16, device="cuda") for _ in range(nmix)]
    h_one = torch.empty((rows, cols), dtype=torch.float16, device="cuda")
    K.layer_norm_ce_mix(dev(x), dev(g), dev(b), 1e-5, p_one, wd, one, out=h_one)
    torch.cuda.synchronize()
    assert torch.equal(h_one, h) and torch.equal(p_one, p_two) and torch.equal(p_one, h)
    for a_, b_ in zip(one, two):
        assert torch.equal(a_, b_)
    want_h = O.layer_norm_ce(x, g, b, 1e-5, rows, 1, cols)
    assert np.abs(host(h_one).astype(np.float32) - want_h.astype(np.float32)).max() <= 4 * 2.0 ** -10 * np.abs(want_h).max()
    for w, o in zip(ws, one):                   # the shift's fp16 steps, on the rows the launch normalised
        assert np.array_equal(host(o).view(np.uint16), OM_gate(host(h_one), w, prev).view(np.uint16))
    # without the copy of the normalised rows
    p_none = dev(prev)
    none = [torch.empty((rows, cols), dtype=torch.float16, device="cuda") for _ in range(nmix)]
    K.layer_norm_ce_mix(dev(x), dev(g), dev(b), 1e-5, p_none, wd, none)
    assert torch.equal(p_none, h) and all(torch.equal(a_, b_) for a_, b_ in zip(none, two))
    with pytest.raises(Exception, match="mixing vector needs its output"):
        lib = K._lib.load()
        K.check(lib.pta_layer_norm_ce_mix(K._p(dev(x)), K._p(dev(g)), K._p(dev(b)), None, K._p(p_none), K._p(wd[0]), K._p(wd[0]), None,
                                          K._p(none[0]), None, None, rows, cols, 1e-5, None))


def test_rwkv_mix_bit_exact_and_wkv(K):
    rng = np.random.default_rng(41)
    B, d = 3, 256
    x = rng.standard_normal((B, d)).astype(np.float16)
    prev = rng.standard_normal((B, d)).astype(np.float16)
    ws = [rng.uniform(0, 1, d).astype(np.float16) for _ in range(3)]
    outs = [torch.empty((B, d), dtype=torch.float16, device="cuda") for _ in range(3)]
    pd = dev(prev)
    K.rwkv_mix(dev(x), pd, [dev(w) for w in ws], outs)
    for w, o in zip(ws, outs):
        assert np.array_equal(host(o).view(np.uint16), OM_gate(x, w, prev).view(np.uint16))
    assert np.array_equal(host(pd), x)
    # WKV: three consecutive steps against the fp32 closed form
    k = [rng.standard_normal((B, d)).astype(np.float16) for _ in range(3)]
    v = [rng.standard_normal((B, d)).astype(np.float16) for _ in range(3)]
    r = [rng.uniform(0, 1, (B, d)).astype(np.float16) for _ in range(3)]
    td = rng.uniform(-8, -1, d).astype(np.float16)
    tf = rng.uniform(-1, 1, d).astype(np.float16)
    num = torch.zeros((B, d), dtype=torch.float32, device="cuda")
    den = torch.zeros_like(num)
    mx = torch.full_like(num, -1e30)
    a = np.zeros((B, d), np.float64); b = np.zeros((B, d), np.float64); p = np.full((B, d), -1e30)
    y = torch.empty((B, d), dtype=torch.float16, device="cuda")
    for t in range(3):
        K.rwkv_wkv(dev(k[t]), dev(v[t]), dev(r[t]), dev(td), dev(tf), num, den, mx, y)
        kk, vv = k[t].astype(np.float64), v[t].astype(np.float64)
        t1 = kk + tf.astype(np.float64)
        M = np.maximum(p, t1)
        out = (np.exp(p - M) * a + np.exp(t1 - M) * vv) / (np.exp(p - M) * b + np.exp(t1 - M))
        p2 = p - np.exp(td.astype(np.float64))
        M2 = np.maximum(p2, kk)
        a, b, p = np.exp(p2 - M2) * a + np.exp(kk - M2) * vv, np.exp(p2 - M2) * b + np.exp(kk - M2), M2
        ref = r[t].astype(np.float64) * out
        assert np.abs(host(y).astype(np.float64) - ref).max() <= 2e-3 * max(1.0, np.abs(ref).max())
        assert np.abs(host(num) - a).max() <= 1e-4 * max(1.0, np.abs(a).max())
        assert np.abs(host(mx) - p).max() <= 1e-5 * np.abs(p).max()


def OM_gate(a, w, b):
    from oracle.models import _gate
    return _gate(a, w, b)


# ---------------------------------------------------------------- selection & loop
@pytest.mark.parametrize("rows,n", [(1, 32000), (16, 50257), (3, 65536), (2, 5)])
def test_argmax(K, rows, n):
    rng = np.random.default_rng(rows + n)
    x = rng.standard_normal((rows, n)).astype(np.float16)
    x[0, [n // 3, n // 2]] = 9.0                       # a tie: the lower index wins
    x[rows // 2, [n - 1, min(7, n - 1), min(8, n - 1)]] = 11.0      # ... across 16-byte vectors and threads, up to the last element
    x[rows - 1, :] = 1.0                               # all equal: index 0 (a later row does not start on a 16-byte boundary when n is odd)
    got = host(K.argmax(dev(x)))
    _, ref = O.topk1(x, -1)
    assert np.array_equal(got, ref[:, 0])


def test_embedding(K):
    rng = np.random.default_rng(4)
    table = rng.standard_normal((100, 64)).astype(np.float16)
    pos = rng.standard_normal((10, 64)).astype(np.float16)
    ids = np.array([3, 99, 0], np.int32)
    assert np.array_equal(host(K.embedding(dev(table), dev(ids))), table[ids])
    p = torch.tensor(7, dtype=torch.int32, device="cuda")
    got = host(K.embedding(dev(table), dev(ids), pos_table=dev(pos), pos=p))
    assert np.array_equal(got, (table[ids] + pos[7]).astype(np.float16))


@pytest.mark.parametrize("early_stop", [False, True])
def test_step_update_matches_loop_simulator(K, early_stop):
    rng = np.random.default_rng(8)
    B, L, pad, eos = 3, 12, 0, 2
    ids = np.full((B, L), pad, np.int32)
    ids[0, :4] = [5, 6, 7, 8]
    ids[1, :2] = [9, 3]
    ids[2, :6] = [4, 4, 2, 4, 4, 4]
    state = O.initial_loop_state(ids, L)
    container = dev(ids.copy())
    mask = dev(state["mask"].copy())
    stop = torch.zeros(B, dtype=torch.int32, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    keep = torch.ones((), dtype=torch.int32, device="cuda")
    ids_out = torch.zeros(B, dtype=torch.int32, device="cuda")
    for it in range(L):
        nxt = rng.integers(1, 6, size=B).astype(np.int32)
        upd = O.step_containers(state, nxt, pad)
        keep_ref = O.step_loop_cond(state, upd, eos, early_stop, B)
        K.step_update(container, mask, stop, step, dev(nxt), ids_out, keep, pad, eos, early_stop)
        assert np.array_equal(host(container), state["container"])
        assert np.array_equal(host(mask), state["mask"])
        assert np.array_equal(host(stop), state["stop_mask"])
        assert int(host(step)) == state["step"]
        assert bool(host(keep)) == keep_ref
        assert np.array_equal(host(ids_out), upd)


# ---------------------------------------------------------------- top-k and sampling
@pytest.mark.parametrize("rows,n,k", [(1, 50257, 5), (3, 1000, 1), (2, 64, 64), (4, 32000, 40)])
def test_topk_matches_a_stable_sort(K, rows, n, k):
    rng = np.random.default_rng(rows + n + k)
    x = rng.standard_normal((rows, n)).astype(np.float16)
    x[:, ::7] = x[:, 3:4]                      # many equal values: ties resolve to the lower index
    vals, ids = K.topk(dev(x), k)
    vals, ids = host(vals), host(ids)
    order = np.argsort(-x.astype(np.float32), axis=1, kind="stable")[:, :k]
    assert np.array_equal(ids, order)
    assert np.array_equal(vals, np.take_along_axis(x, order, axis=1))


def test_topk_guards_and_take_column(K):
    x = dev(np.zeros((2, 8), np.float16))
    with pytest.raises(ValueError):
        K.topk(x, 9)
    with pytest.raises(ValueError):
        K.topk(x, 0)
    cand = dev(np.arange(12, dtype=np.int32).reshape(3, 4))
    for pick, col in ((0, 0), (3, 3), (7, 3), (-2, 0)):     # out-of-range picks are clamped
        got = host(K.take_column(cand, dev(np.array([pick], np.int32))))
        assert np.array_equal(got, np.arange(12).reshape(3, 4)[:, col])


# ---------------------------------------------------------------- BeamSearch, KVCachePipeline transpose
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("B,beam,V,L", [(2, 4, 1000, 12), (1, 1, 37, 5), (3, 8, 32000, 20), (2, 64, 80, 9)])
def test_beam_search_step_bit_exact(K, dtype, B, beam, V, L):
    """Ids, flat candidate indices, both containers bit for bit over more steps than the container has rows
    (the steps beyond it only re-gather), fp16 logits with many equal scores included."""
    rng = np.random.default_rng(B * 1000 + beam + V)
    tdt = torch.float16 if dtype == np.float16 else torch.float32
    hyp_ref = rng.integers(-5, 5, size=(B, L, beam)).astype(np.int32)      # whatever the caller left there
    prob_ref = rng.standard_normal((B, beam)).astype(dtype)
    hyp, prob = dev(hyp_ref), dev(prob_ref)
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    ws = torch.empty(K._lib.load().pta_beam_search_workspace_bytes(B, beam), dtype=torch.uint8, device="cuda")
    for it in range(L + 2):
        # log-probabilities of a peaked distribution; in fp16 many of them coincide
        logits = np.log(rng.dirichlet(np.full(V, 0.3), size=(B, beam)) + 1e-9).astype(dtype)
        nxt_ref, best_ref, hyp_ref, prob_ref = O.beam_search_step(logits, hyp_ref, prob_ref, it, beam)
        step.fill_(it)
        nxt, best = K.beam_search_step(dev(logits).to(tdt), hyp, prob, step, ws)
        assert np.array_equal(host(nxt), nxt_ref), f"next_id differs at step {it}"
        assert np.array_equal(host(best), best_ref), f"global_best_id differs at step {it}"
        assert np.array_equal(host(hyp), hyp_ref), f"hyp_container differs at step {it}"
        assert np.array_equal(host(prob).view(np.uint8), prob_ref.view(np.uint8)), f"prob_container differs at step {it}"


def test_beam_search_guards(K):
    z = lambda *s, dt=torch.float16: torch.zeros(s, dtype=dt, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        K.beam_search_step(z(2, 5), z(1, 4, 2, dt=torch.int32), z(1, 2), step)            # rank of logits
    with pytest.raises(ValueError):
        K.beam_search_step(z(1, 2, 5), z(1, 4, 3, dt=torch.int32), z(1, 2), step)         # beam sizes differ
    with pytest.raises(ValueError):
        K.beam_search_step(z(1, 6, 5), z(1, 4, 6, dt=torch.int32), z(1, 6), step)         # beam > vocabulary
    with pytest.raises(ValueError):
        K.beam_search_step(z(1, 2, 5), z(1, 4, 2, dt=torch.int32), z(1, 2, dt=torch.float32), step)


@pytest.mark.parametrize("shape,max_len,max_bps,dtype", [((2, 2, 1, 16), 4, 3, np.float16), ((3, 1, 40), 130, 2, np.float16),
                                                           ((2, 1, 1, 128), 70, 1, np.uint8), ((1, 5, 1, 33), 65, 2, np.float32)])
def test_kv_cache_pipeline_seq_last(K, shape, max_len, max_bps, dtype):
    """transpose = 1: the registers keep the sequence as their last axis and shift in place; output and stored
    registers against the oracle bit for bit, over more steps than the registers hold, then a second generation
    from step 0 (which zeroes every register)."""
    rng = np.random.default_rng(max_len + max_bps)
    ref_op = O.KVCachePipeline(max_len, max_bps, transpose=True)
    outer, inner = int(np.prod(shape[:-2])), shape[-1]
    tdt = {np.float16: torch.float16, np.uint8: torch.uint8, np.float32: torch.float32}[dtype]
    caches = torch.full((max_bps, outer, inner, max_len), 5, dtype=tdt, device="cuda")     # stale contents before step 0
    out = torch.empty(shape[:-2] + (max_len, inner), dtype=tdt, device="cuda")
    step = torch.zeros((), dtype=torch.int32, device="cuda")
    for it in list(range(max_bps * (max_len + 2))) + [0, 1, 2, 3]:
        upd = rng.integers(0, 255, size=shape).astype(np.uint8) if dtype == np.uint8 else rng.standard_normal(shape).astype(dtype)
        ref = ref_op(it, upd)
        step.fill_(it)
        K.kv_cache_pipeline_seq_last(caches, out, dev(upd), step, outer, max_len, inner, max_bps)
        assert np.array_equal(host(out), ref), f"output differs at step {it}"
        stored = np.stack([c.reshape(outer, inner, max_len) for c in ref_op.stored()])
        assert np.array_equal(host(caches), stored), f"stored registers differ at step {it}"


# ---------------------------------------------------------------- FP8 x FP8 on the FP8 matrix instruction
def _f143_case(rng, M, Kdim, N, scale, specials):
    """Random F143 bytes for both operands; with `specials`, the three codes whose value is not half of the OCP
    value of the same bits (+240, -240 and, optionally, NaN) are placed in weights and activations."""
    x8 = O.f8_encode(rng.standard_normal((M, Kdim)).astype(np.float16), "F143", scale)
    w8 = O.f8_encode((rng.standard_normal((Kdim, N)) * 0.02).astype(np.float32), "F143", scale)
    if specials:
        w8[3, 0], w8[Kdim - 1, N - 1], w8[130, min(17, N - 1)] = 0x7F, 0xFF, 0x7F
        x8[0, 5], x8[M - 1, Kdim - 2] = 0x7F, 0xFF
        w8[7, 1], x8[0, 200] = 0x01, 0x81                   # the smallest subnormals
    return x8, w8


@pytest.mark.parametrize("M,Kdim,N", [(1, 4096, 48), (8, 4096, 8192), (16, 1160, 13696), (5, 13696, 4096)])
@pytest.mark.parametrize("specials", [False, True])
def test_fp8_products_on_the_fp8_matrix_instruction(K, M, Kdim, N, specials):
    """Both operands F143, up to 16 rows: the bytes go to the FP8 instruction as they are.  Left-hand side as bytes
    and as fp16 values on the grid; one, two and three channel blocks per workgroup; a ragged last feature tile;
    +-240 and subnormals in both operands (steps holding +-240 are multiplied through exact fp16 decodes)."""
    rng = np.random.default_rng(M + Kdim + N)
    scale = -1
    x8, w8 = _f143_case(rng, M, Kdim, N, scale, specials)
    sd = dev(np.array([scale], np.int32))
    fw = K.F8Weight(dev(w8), sd, "F143", kn=True)
    ref = O.fp8_matmul(x8, w8, [scale], [scale], "F143", "F143")
    tol = 2.0 ** -10 * np.abs(ref.astype(np.float64)).max()                    # one fp16 rounding of the largest output
    got = host(K.fp8_gemm(dev(x8), fw, K.fp8_gemm_workspace(M, Kdim, "cuda"), x_scale=sd, x_format="F143"))
    assert np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() <= tol
    xg = dev(O.f8_decode(x8, "F143", 0, np.float16))                           # the same activations as grid values
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    K.linear(xg, [fw], [out], x_scale=sd)
    assert np.abs(host(out).astype(np.float64) - ref.astype(np.float64)).max() <= tol


def test_fp8_products_pair_multi_and_nan(K):
    rng = np.random.default_rng(77)
    M, Kdim, N, scale = 8, 4096, 13696, -2
    sd = dev(np.array([scale], np.int32))
    x8, wg8 = _f143_case(rng, M, Kdim, N, scale, True)
    _, wu8 = _f143_case(rng, M, Kdim, N, scale, True)
    xg = dev(O.f8_decode(x8, "F143", 0, np.float16))
    g, u = K.F8Weight(dev(wg8), sd, "F143", kn=True), K.F8Weight(dev(wu8), sd, "F143", kn=True)
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    K.linear(xg, [g, u], [out, out], x_scale=sd, swiglu=True)
    rg, ru = (O.fp8_matmul(x8, w, [scale], [scale]) for w in (wg8, wu8))
    ref = (ru * O.swish(rg)).astype(np.float16)
    assert rel_err(host(out), ref) <= 1e-2
    # two matrices of different widths in one launch, each with a bias
    _, w2 = _f143_case(rng, M, Kdim, 512, scale, True)
    b1, b2 = rng.standard_normal(N).astype(np.float16), rng.standard_normal(512).astype(np.float16)
    o1, o2 = torch.empty((M, N), dtype=torch.float16, device="cuda"), torch.empty((M, 512), dtype=torch.float16, device="cuda")
    K.linear(xg, [g, K.F8Weight(dev(w2), sd, "F143", kn=True)], [o1, o2], biases=[dev(b1), dev(b2)], x_scale=sd)
    assert rel_err(host(o1), (rg + b1).astype(np.float16)) <= 1e-2
    assert rel_err(host(o2), (O.fp8_matmul(x8, w2, [scale], [scale]) + b2).astype(np.float16)) <= 1e-2
    # the NaN code: as a weight it poisons its output channel, as an activation its row - and nothing else
    wn, xn = wg8.copy(), x8.copy()
    wn[900, 33] = 0x80
    xn[2, 1000] = 0x80
    got = host(K.fp8_gemm(dev(xn), K.F8Weight(dev(wn), sd, "F143", kn=True), K.fp8_gemm_workspace(M, Kdim, "cuda"),
                          x_scale=sd, x_format="F143"))
    with np.errstate(invalid="ignore"):
        ref = O.fp8_matmul(xn, wn, [scale], [scale])
    assert np.array_equal(np.isnan(got), np.isnan(ref)) and np.isnan(ref[2]).all() and np.isnan(ref[:, 33]).all()
    ok = ~np.isnan(ref)
    assert np.abs(got[ok].astype(np.float64) - ref[ok].astype(np.float64)).max() <= 2.0 ** -10 * np.abs(ref[ok].astype(np.float64)).max()


@pytest.mark.parametrize("M,Kdim,N", [(M, Kdim, N) for M in (48, 65, 200, 256, 1024)
                                      for Kdim, N in ((4096, 4096), (1160, 8192), (2048, 512), (1024, 100))] + [(2048, 1024, 8192)])
@pytest.mark.parametrize("specials", [False, True])
def test_fp8_products_of_many_rows_on_the_fp8_matrix_instruction(K, M, Kdim, N, specials):
    """Both operands F143, more than 64 rows (a prompt pass): the 16x16x128 FP8 instruction with the activations turned
    into bytes on their way to LDS.  The shapes reach all five forms of the kernel - row blocks of 128 rows (2048 x
    1024 x 8192), of 64 (1024 x 1160 x 8192; with K in halves 1024 x 4096 x 4096) and of 32 (200 x 1160 x 8192; in
    halves 200 x 4096 x 4096) -, ragged last row blocks (65, 200) and feature tiles (1160), a channel count outside
    the kernel's tiles (100) and a row count below it (48), which take the fp16 instruction's paths; +-240, stretches
    of them, and the smallest subnormals in both operands.  Left-hand side as fp16 values on the grid and as bytes;
    within one fp16 rounding of the largest output of the oracle's product."""
    rng = np.random.default_rng(M + Kdim + N)
    scale = -1
    x8, w8 = _f143_case(rng, M, Kdim, N, scale, specials)
    if specials:
        x8[M // 2, :64] = 0x7F                 # a stretch of saturated activations, and rows of them in other row groups
        x8[M - 1, Kdim - 40:] = 0xFF
        x8[16, 129] = 0xFF
    sd = dev(np.array([scale], np.int32))
    fw = K.F8Weight(dev(w8), sd, "F143", kn=True)
    ref = O.fp8_matmul(x8, w8, [scale], [scale], "F143", "F143")
    tol = 2.0 ** -10 * np.abs(ref.astype(np.float64)).max()
    xg = dev(O.f8_decode(x8, "F143", 0, np.float16))
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    K.linear(xg, [fw], [out], x_scale=sd)
    assert np.abs(host(out).astype(np.float64) - ref.astype(np.float64)).max() <= tol
    got = host(K.fp8_gemm(dev(x8), fw, K.fp8_gemm_workspace(M, Kdim, "cuda"), x_scale=sd, x_format="F143"))
    assert np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() <= tol


@pytest.mark.parametrize("M", [100, 200])
def test_fp8_products_of_many_rows_pair_multi_and_nan(K, M):
    rng = np.random.default_rng(79 + M)
    Kdim, N, scale = 2048, 1408, -2
    sd = dev(np.array([scale], np.int32))
    x8, wg8 = _f143_case(rng, M, Kdim, N, scale, True)
    _, wu8 = _f143_case(rng, M, Kdim, N, scale, True)
    xg = dev(O.f8_decode(x8, "F143", 0, np.float16))
    g, u = K.F8Weight(dev(wg8), sd, "F143", kn=True), K.F8Weight(dev(wu8), sd, "F143", kn=True)
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    K.linear(xg, [g, u], [out, out], x_scale=sd, swiglu=True)
    rg, ru = (O.fp8_matmul(x8, w, [scale], [scale]) for w in (wg8, wu8))
    ref = (ru * O.swish(rg)).astype(np.float16)
    assert rel_err(host(out), ref) <= 1e-2
    # two matrices of different widths in one launch, each with a bias; a residual on a single one
    _, w2 = _f143_case(rng, M, Kdim, 512, scale, True)
    b1, b2 = rng.standard_normal(N).astype(np.float16), rng.standard_normal(512).astype(np.float16)
    o1, o2 = torch.empty((M, N), dtype=torch.float16, device="cuda"), torch.empty((M, 512), dtype=torch.float16, device="cuda")
    K.linear(xg, [g, K.F8Weight(dev(w2), sd, "F143", kn=True)], [o1, o2], biases=[dev(b1), dev(b2)], x_scale=sd)
    assert rel_err(host(o1), (rg + b1).astype(np.float16)) <= 1e-2
    assert rel_err(host(o2), (O.fp8_matmul(x8, w2, [scale], [scale]) + b2).astype(np.float16)) <= 1e-2
    # the NaN code: as a weight it poisons its output channel, as an activation its row - and nothing else
    wn, xn = wg8.copy(), x8.copy()
    wn[900, 33] = 0x80
    xn[M - 2, 1000] = 0x80
    got = host(K.fp8_gemm(dev(xn), K.F8Weight(dev(wn), sd, "F143", kn=True), K.fp8_gemm_workspace(M, Kdim, "cuda"),
                          x_scale=sd, x_format="F143"))
    with np.errstate(invalid="ignore"):
        ref = O.fp8_matmul(xn, wn, [scale], [scale])
    assert np.array_equal(np.isnan(got), np.isnan(ref)) and np.isnan(ref[M - 2]).all() and np.isnan(ref[:, 33]).all()
    ok = ~np.isnan(ref)
    assert np.abs(got[ok].astype(np.float64) - ref[ok].astype(np.float64)).max() <= 2.0 ** -10 * np.abs(ref[ok].astype(np.float64)).max()


# ---------------------------------------------------------------- more than 64 rows
@pytest.mark.parametrize("M", [65, 128, 200, 256, 600, 1024])
@pytest.mark.parametrize("Kdim,N", [(4096, 4096), (1160, 8192), (11008, 4096), (512, 100)])
def test_w4a16_gemm_up_to_256_rows(K, M, Kdim, N):
    """More than 64 rows: up to 128 the kernel that keeps the activation fragments in registers, beyond them the
    kernel that takes 128-row panels through LDS and the weights straight into registers;
    with and without the K split that a workspace allows; 1160 features = a ragged last tile; 200 and 600 rows = a
    ragged last row block, and for channel counts that do not divide into the workgroup tiles (100) the 64-row
    paths over the rows in turn.  Bias and a residual that aliases the output; the residual alone (the epilogue
    that moves whole vectors)."""
    x, packed, scale = _w4_case(M + Kdim + N, M, Kdim, N)
    rng = np.random.default_rng(M * N)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    w = K.W4Weight(dev(packed), dev(scale))
    ref = ((O.w4a16_matmul(x, packed, scale) + bias).astype(np.float16) + res).astype(np.float16)
    assert rel_err(host(K.w4a16_gemm(dev(x), w, bias=dev(bias), residual=dev(res))), ref) <= 1e-2
    ws = K.linear_workspace(M, N, "cuda")
    ws.fill_(0xFF)
    y = dev(res.copy())
    K.w4a16_gemm(dev(x), w, bias=dev(bias), residual=y, out=y, workspace=ws)
    assert rel_err(host(y), ref) <= 1e-2
    ref = (O.w4a16_matmul(x, packed, scale) + res).astype(np.float16)
    y = dev(res.copy())
    K.w4a16_gemm(dev(x), w, residual=y, out=y)
    assert rel_err(host(y), ref) <= 1e-2


def test_w4a16_gemm_most_rows_few_channels_exact_integers(K):
    """4096 rows (the most a launch takes) and 256 channels: a workgroup of the panel kernel in which half the waves
    have no channel blocks and only help to bring the rows in; 3000 rows = a ragged last panel."""
    rng = np.random.default_rng(77)
    for M in (4096, 3000):
        Kdim, N = 512, 256
        x = rng.integers(-2, 3, size=(M, Kdim)).astype(np.float16)
        q = rng.integers(-8, 8, size=(N, Kdim))
        w = K.W4Weight(dev(O.pack_int4(q)), dev(np.ones(N, np.float16)))
        assert np.array_equal(host(K.w4a16_gemm(dev(x), w)).astype(np.int64), x.astype(np.int64) @ q.T.astype(np.int64))


def test_w4a16_gemm_last_round_of_tiles_in_a_launch_of_its_own(K):
    """More workgroup tiles than compute units with a last round that fills at most half of them: the channel groups
    of the whole rounds run in one launch, the rest in a second one with K in halves inside the workgroup (its
    units start in the middle of the matrices).  11008 channels at 2048 rows (352 tiles of 128 rows x 512 channels),
    the SwiGLU pair at 1024 rows (344 tiles), and three matrices in one launch at 2048 rows."""
    rng = np.random.default_rng(91)
    Kdim = 1024
    mats = [(rng.integers(-128, 128, size=(n, Kdim // 2), dtype=np.int8), rng.uniform(0.005, 0.02, size=(n,)).astype(np.float16))
            for n in (11008, 11008, 4096, 4096)]
    ws = [K.W4Weight(dev(p), dev(s_)) for p, s_ in mats]
    x = rng.standard_normal((2048, Kdim)).astype(np.float16)
    assert rel_err(host(K.w4a16_gemm(dev(x), ws[0])), O.w4a16_matmul(x, *mats[0])) <= 1e-2
    for (p, s_), o in zip(mats[1:], K.w4a16_gemm_multi(dev(x), ws[1:])):
        assert rel_err(host(o), O.w4a16_matmul(x, p, s_)) <= 1e-2
    x = x[:1024].copy()
    got = host(K.w4a16_gemm_swiglu(dev(x), ws[0], ws[1]))
    ref = (O.w4a16_matmul(x, *mats[1]) * O.swish(O.w4a16_matmul(x, *mats[0]))).astype(np.float16)
    assert rel_err(got, ref) <= 1e-2


def test_gemm_up_to_256_rows_exact_integers_pair_and_other_formats(K):
    rng = np.random.default_rng(61)
    for M in (96, 256, 520):
        Kdim, N = 1024, 8192
        x = rng.integers(-2, 3, size=(M, Kdim)).astype(np.float16)
        q = rng.integers(-8, 8, size=(N, Kdim))
        w = K.W4Weight(dev(O.pack_int4(q)), dev(np.ones(N, np.float16)))
        assert np.array_equal(host(K.w4a16_gemm(dev(x), w)).astype(np.int64), x.astype(np.int64) @ q.T.astype(np.int64))
        # SwiGLU pair, three matrices in one launch
        xr = rng.standard_normal((M, Kdim)).astype(np.float16)
        mats = [(rng.integers(-128, 128, size=(n, Kdim // 2), dtype=np.int8), rng.uniform(0.005, 0.02, size=(n,)).astype(np.float16))
                for n in (11008, 11008, 4096, 2048)]
        ws = [K.W4Weight(dev(p), dev(s_)) for p, s_ in mats]
        got = host(K.w4a16_gemm_swiglu(dev(xr), ws[0], ws[1]))
        ref = (O.w4a16_matmul(xr, *mats[1]) * O.swish(O.w4a16_matmul(xr, *mats[0]))).astype(np.float16)
        assert rel_err(got, ref) <= 1e-2
        for (p, s_), o in zip(mats[1:], K.w4a16_gemm_multi(dev(xr), ws[1:])):
            assert rel_err(host(o), O.w4a16_matmul(xr, p, s_)) <= 1e-2
        # fp16 and FP8 weights
        wf = (rng.standard_normal((768, Kdim)) * 0.05).astype(np.float16)
        assert rel_err(host(K.f16_gemm(dev(xr), K.F16Weight(dev(wf)))), O.matmul(xr, wf.T.copy())) <= 1e-2
        w8 = O.f8_encode((rng.standard_normal((Kdim, 4096)) * 0.02).astype(np.float32), "F143", -1)
        fw = K.F8Weight(dev(w8), dev(np.array([-1], np.int32)), "F143", kn=True)
        assert rel_err(host(K.fp8_gemm(dev(xr), fw, K.fp8_gemm_workspace(M, Kdim, "cuda"))), O.fp8_matmul(xr, w8, [-1], [-1])) <= 1e-2
    with pytest.raises(ValueError):
        K.w4a16_gemm(dev(rng.standard_normal((4097, 1024)).astype(np.float16)), w)
