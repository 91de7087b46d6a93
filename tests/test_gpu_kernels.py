"""HIP kernels against the CPU oracle, through the C ABI.

Follows ferrotensor-backend/tests/gpu_kernels.rs: every kernel on seeded
inputs at the reference's shapes (MATMUL_SHAPES :234-246, SMOLLM2_PROJECTIONS
:966-982, row kernels, masked CE, AdamW), compared with the oracle within
|a-e| <= 1e-4 + 1e-3*|e| (f32) and bit-exactly for integer/index work.
"""
import numpy as np
import pytest

from oracle import cpu
from oracle import reference_step as rs
from tests.gpu_util import assert_close, make_ctx

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    ctx, eng = make_ctx()
    yield ctx, eng
    ctx.close()


def rnd(seed, *shape, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(np.float32)


def up(ctx, x):
    from ferrotensor_amd import UnifiedTensor
    return UnifiedTensor.new(ctx, x, list(x.shape))


def empty(ctx, *shape):
    from ferrotensor_amd import UnifiedTensor
    return UnifiedTensor.empty(ctx, list(shape))


MATMUL_SHAPES = [(1, 1, 1), (1, 7, 1), (3, 5, 7), (16, 16, 16), (17, 33, 9), (64, 64, 64), (65, 1, 130),
                 (127, 129, 65), (1, 512, 300), (300, 512, 1), (256, 384, 128), (130, 70, 200), (256, 96, 320),
                 # the DMA-fed f32 kernels: ragged last tiles, rows that are no multiple of 4, one and many K tiles
                 (200, 128, 132), (132, 64, 260), (130, 64, 256), (260, 2048, 128), (129, 96, 131), (2048, 576, 1536), (256, 4096, 192),
                 # the kernel microbenchmark's weight-gradient product x^T @ dY: M = in, K = rows, N = out
                 (576, 2048, 1536)]

# GEMM tolerance of the reference's f64 comparisons (gpu_kernels.rs:989-1084): 1e-3 + 1e-4*|want|
# for N(0,1) operands; the oracle itself adds in f32, so compare against f64 here.


def f64_mm(a, b):
    return a.astype(np.float64) @ b.astype(np.float64)


@pytest.mark.parametrize("M,K,N", MATMUL_SHAPES)
def test_matmul_layouts_match_cpu(g, M, K, N):
    ctx, eng = g
    a, b = rnd(M * 7 + K, M, K), rnd(N * 3 + K, K, N)
    want = f64_mm(a, b)
    out = empty(ctx, M, N)
    eng.matmul(ctx, up(ctx, a), up(ctx, b), out)
    assert_close(f"matmul {M}x{K}x{N}", out.to_numpy(), want, atol=1e-3, rtol=1e-4)
    out = empty(ctx, M, N)
    eng.matmul_bt(ctx, up(ctx, a), up(ctx, np.ascontiguousarray(b.T)), out)
    assert_close(f"matmul_bt {M}x{K}x{N}", out.to_numpy(), want, atol=1e-3, rtol=1e-4)
    out = empty(ctx, M, N)
    eng.matmul_at(ctx, up(ctx, np.ascontiguousarray(a.T)), up(ctx, b), out)
    assert_close(f"matmul_at {M}x{K}x{N}", out.to_numpy(), want, atol=1e-3, rtol=1e-4)
    # and against the oracle's own f32 product
    assert_close(f"matmul vs oracle {M}x{K}x{N}", out.to_numpy(), cpu.matmul(a, b), atol=1e-3, rtol=1e-4)


# every row of gpu_kernels.rs:966-982
SMOLLM2_PROJECTIONS = [("135M q/o", 576, 576), ("135M k/v", 576, 192), ("135M fused qkv", 576, 960),
                       ("135M gate/up", 576, 1536), ("135M down", 1536, 576), ("135M lm_head", 576, 49152),
                       ("360M q/o", 960, 960), ("360M k/v", 960, 320), ("360M fused qkv", 960, 1600),
                       ("360M gate/up", 960, 2560), ("360M down", 2560, 960), ("360M lm_head", 960, 49152),
                       ("1.7B q/k/v/o", 2048, 2048), ("1.7B gate/up", 2048, 8192), ("1.7B down", 8192, 2048)]


@pytest.mark.parametrize("name,K,N", SMOLLM2_PROJECTIONS)
@pytest.mark.parametrize("M", [31, 256])
def test_f16_weight_projections(g, name, K, N, M):
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    a, w = rnd(K + N, M, K), rnd(K * 2 + N, K, N, scale=0.05)
    w16 = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N])
    wr = cpu.round_f16(w)
    out = empty(ctx, M, N)
    eng.matmul_f16b(ctx, up(ctx, a), w16, out)
    assert_close(f"{name} matmul_f16b", out.to_numpy(), f64_mm(a, wr), atol=1e-3, rtol=1e-4)
    # input gradient: g[M,N] @ w[K,N]^T
    gy = rnd(7, M, N)
    dx = empty(ctx, M, K)
    eng.matmul_bt_f16b(ctx, up(ctx, gy), w16, dx)
    assert_close(f"{name} matmul_bt_f16b", dx.to_numpy(), f64_mm(gy, wr.T), atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("name,M,K,N", [("1.7B gate/up, 8 x 1024 rows", 8192, 2048, 8192),
                                        ("1.7B down, 8 x 1024 rows", 8192, 8192, 2048),
                                        ("360M lm_head on the supervised rows of the headline batch", 1446, 960, 49152)])
def test_projections_at_the_row_counts_of_the_full_batches(g, name, M, K, N):
    """The GEMMs of the 1.7B-shaped step at its real row count (M = 8192: thousands of tiles per launch) and
    the vocabulary head (the 128x128 tile): forward and input gradient, sampled rows against f64 (the full
    f64 product of these shapes would take the CPU minutes; every row block and column panel is sampled)."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    rng = np.random.default_rng(K + N)
    a = rng.standard_normal((M, K), dtype=np.float32)
    w = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.05)
    w16 = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N])
    wr = cpu.round_f16(w)
    del w
    rows = np.unique(np.concatenate([np.arange(0, M, 61), [M - 1, M - 2, 63, 64, 127, 128]]))
    out = empty(ctx, M, N)
    eng.matmul_f16b(ctx, up(ctx, a), w16, out)
    assert_close(f"{name} matmul_f16b", out.to_numpy()[rows], f64_mm(a[rows], wr), atol=2e-3, rtol=1e-4)
    del out
    gy = rng.standard_normal((M, N), dtype=np.float32)
    dx = empty(ctx, M, K)
    eng.matmul_bt_f16b(ctx, up(ctx, gy), w16, dx)
    bar = 2e-3 * max(1.0, np.sqrt(N / 2048.0))     # sums of N products of N(0,1) x N(0,0.05): spread grows as sqrt(N)
    assert_close(f"{name} matmul_bt_f16b", dx.to_numpy()[rows], f64_mm(gy[rows], wr.T), atol=bar, rtol=1e-4)


# K loops of one, two and three 32-wide tiles (the pipeline's prologue alone, with the clamped re-read after the
# last tile), and the shortest shares split-K ever makes (a share holds at least 4 K tiles: K = 256 -> 4 + 4,
# K = 288 -> 5 + 4, K = 512 -> four shares of 4; K = 832 -> three shares of 5 + 4 + 4 tile pairs on eight waves).
SHORT_K = [32, 64, 96]
SMALLEST_SHARES_K = [256, 288, 512, 832]


@pytest.mark.parametrize("K", SHORT_K + SMALLEST_SHARES_K)
@pytest.mark.parametrize("M,N", [(256, 192), (31, 960), (130, 128)])
def test_f16_weight_products_with_short_k_and_smallest_split_shares(g, M, N, K):
    """(256, 192) and (130, 128) are a dozen 64x64 tiles or fewer, so K >= 256 is split over workgroups;
    (31, 960) is one ragged row block."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    a, w = rnd(K + N + M, M, K), rnd(K * 2 + N, K, N, scale=0.05)
    w16 = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N])
    wr = cpu.round_f16(w)
    out = empty(ctx, M, N)
    eng.matmul_f16b(ctx, up(ctx, a), w16, out)
    assert_close(f"matmul_f16b {M}x{K}x{N}", out.to_numpy(), f64_mm(a, wr), atol=1e-3, rtol=1e-4)
    # the other operand layout: g[M, N'] @ w[K', N']^T with the short loop over N' = K
    w2 = rnd(K * 3 + N, N, K, scale=0.05)
    w2_16 = UnifiedTensor.from_f32_as_f16(ctx, w2, [N, K])
    dx = empty(ctx, M, N)
    eng.matmul_bt_f16b(ctx, up(ctx, a), w2_16, dx)
    assert_close(f"matmul_bt_f16b {M}x{K}x{N}", dx.to_numpy(), f64_mm(a, cpu.round_f16(w2).T), atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("K", [64, 96, 256, 288, 512])
@pytest.mark.parametrize("M,N", [(256, 128), (132, 260)])
def test_f32_products_with_short_k_and_smallest_split_shares(g, M, N, K):
    """The DMA-fed f32 kernel takes K >= 64 (two tiles); (256, 128) is 8 tiles of 64x64, so K >= 256 is split
    into shares of 4 and 5 tiles; (132, 260) has ragged last tiles both ways. All three operand layouts."""
    ctx, eng = g
    a, b = rnd(M * 7 + K, M, K), rnd(N * 3 + K, K, N)
    want = f64_mm(a, b)
    out = empty(ctx, M, N)
    eng.matmul(ctx, up(ctx, a), up(ctx, b), out)
    assert_close(f"matmul {M}x{K}x{N}", out.to_numpy(), want, atol=1e-3, rtol=1e-4)
    out = empty(ctx, M, N)
    eng.matmul_bt(ctx, up(ctx, a), up(ctx, np.ascontiguousarray(b.T)), out)
    assert_close(f"matmul_bt {M}x{K}x{N}", out.to_numpy(), want, atol=1e-3, rtol=1e-4)
    out = empty(ctx, M, N)
    eng.matmul_at(ctx, up(ctx, np.ascontiguousarray(a.T)), up(ctx, b), out)
    assert_close(f"matmul_at {M}x{K}x{N}", out.to_numpy(), want, atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("M,K,N", [(2048, 960, 1600), (2000, 512, 1600), (2048, 960, 1664)])
def test_tile_counts_just_above_a_multiple_of_the_cu_count(g, M, K, N):
    """800 (or 832) tiles of 64x64 on 256 CUs: the last 32 (64) tiles of the order are shared out along K over
    8 or 4 workgroups each and added by a second kernel. Plain product, product with residual and rank-8 term,
    and the input-gradient layout; 2000 rows: a ragged last row block among the shared tiles."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    a, w = rnd(K + N, M, K), rnd(K * 2 + N, K, N, scale=0.05)
    w16 = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N])
    wr = cpu.round_f16(w)
    out = empty(ctx, M, N)
    eng.matmul_f16b(ctx, up(ctx, a), w16, out)
    want = f64_mm(a, wr)
    assert_close("matmul_f16b", out.to_numpy(), want, atol=1e-3, rtol=1e-4)
    t, b2, res = rnd(3, M, 8), rnd(4, 8, N), rnd(5, M, N)
    out = empty(ctx, M, N)
    eng.lora_linear(ctx, up(ctx, a), w16, up(ctx, t), up(ctx, b2), out, up(ctx, res))
    assert_close("lora_linear + residual", out.to_numpy(), want + f64_mm(t, b2) + res, atol=1e-3, rtol=1e-4)
    w2 = rnd(K * 3 + N, N, K, scale=0.05)
    w2_16 = UnifiedTensor.from_f32_as_f16(ctx, w2, [N, K])
    dx = empty(ctx, M, N)
    eng.matmul_bt_f16b(ctx, up(ctx, a), w2_16, dx)
    assert_close("matmul_bt_f16b", dx.to_numpy(), f64_mm(a, cpu.round_f16(w2).T), atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("M,K,N", [(1536, 2560, 960), (2048, 1024, 960), (1472, 2048, 896)])
def test_long_k_products_on_eight_waves(g, M, K, N):
    """320 to 512 output tiles of 64x64 and K >= 1024: the workgroup's eight waves share the K loop
    in pairs of tiles (both operand layouts; 1472 rows: a ragged last row block)."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    a, w = rnd(K + N, M, K), rnd(K * 2 + N, K, N, scale=0.05)
    w16 = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N])
    wr = cpu.round_f16(w)
    out = empty(ctx, M, N)
    eng.matmul_f16b(ctx, up(ctx, a), w16, out)
    assert_close("matmul_f16b", out.to_numpy(), f64_mm(a, wr), atol=2e-3, rtol=1e-4)
    # the other layout contracts over the weight's second dimension: w2 [N, K], g [M, K] -> [M, N]
    w2 = rnd(K + 3 * N, N, K, scale=0.05)
    w2_16 = UnifiedTensor.from_f32_as_f16(ctx, w2, [N, K])
    gy = rnd(9, M, K)
    dx = empty(ctx, M, N)
    eng.matmul_bt_f16b(ctx, up(ctx, gy), w2_16, dx)
    assert_close("matmul_bt_f16b", dx.to_numpy(), f64_mm(gy, cpu.round_f16(w2).T), atol=2e-3, rtol=1e-4)


def test_f16_upload_is_bit_exact(g):
    from ferrotensor_amd import DType, UnifiedTensor
    ctx, _ = g
    x = np.concatenate([rnd(1, 4097), rnd(2, 100) * 1e-6, rnd(3, 100) * 1e5,
                        np.array([0.0, -0.0, 65504.0, 65520.0, 1e9, 5.9604645e-08, 2.9802322e-08], np.float32)])
    t = UnifiedTensor.from_f32_as_f16(ctx, x, [x.size])
    got = t.to_vec(ctx, np.uint16)
    np.testing.assert_array_equal(got, cpu.pack_f16(x))
    m = rnd(4, 37, 53)
    tt = UnifiedTensor.from_f32_transposed(ctx, m, 37, 53, DType.FP16)
    assert tt.shape == [53, 37]
    np.testing.assert_array_equal(tt.to_vec(ctx, np.uint16), cpu.pack_f16(np.ascontiguousarray(m.T)).reshape(-1))
    tf = UnifiedTensor.from_f32_transposed(ctx, m, 37, 53, DType.FP32)
    np.testing.assert_array_equal(tf.to_numpy(), m.T)


@pytest.mark.parametrize("M,K,N,r", [(64, 32, 48, 4), (256, 576, 1536, 8), (100, 960, 320, 8), (96, 64, 40, 16),
                                     # ranks the vector kernels do not take (not 4, 8 or 16): the general route
                                     (96, 64, 40, 2), (256, 576, 1536, 32), (70, 96, 200, 1), (128, 192, 64, 12),
                                     (2048, 576, 1536, 8)])  # the last: the kernel-microbench GEMM, full size
@pytest.mark.parametrize("f16", [False, True])
def test_fused_lora_linear_forward_and_backward(g, M, K, N, r, f16):
    """Linear::project_2d and its backward (graph/src/lib.rs:112-126; autograd MatMulNode/ScaleNode)."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    x, w = rnd(1, M, K), rnd(2, K, N, scale=0.05)
    A, B = rnd(3, K, r, scale=0.1), rnd(4, r, N, scale=0.1)
    dy = rnd(5, M, N)
    s = 2.0
    wr = cpu.round_f16(w) if f16 else w
    lin = rs.Linear(weight=wr, lora_a=A, lora_b=B, alpha=s * r, rank=r)
    cache, grads = {}, {}
    want_y = lin.forward(x, cache)
    want_dx = lin.backward(dy, cache, True, False, grads, "l")

    wt = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N]) if f16 else up(ctx, w)
    xt, At, Bt, dyt = up(ctx, x), up(ctx, A), up(ctx, B), up(ctx, dy)
    t = empty(ctx, M, r)
    eng.lora_down(ctx, xt, At, t, s)
    assert_close("x@A*s", t.to_numpy(), cache["temp"], atol=1e-3, rtol=1e-4)
    y = empty(ctx, M, N)
    eng.lora_linear(ctx, xt, wt, t, Bt, y)
    assert_close("lora_linear", y.to_numpy(), want_y, atol=1e-3, rtol=1e-4)
    dt = empty(ctx, M, r)
    eng.lora_grad_down(ctx, dyt, Bt, dt, s)
    dx = empty(ctx, M, K)
    eng.lora_linear_dx(ctx, dyt, wt, dt, At, dx)
    assert_close("lora_linear_dx", dx.to_numpy(), want_dx, atol=2e-3, rtol=1e-4)
    # residual added in the epilogue: a separate tensor, and the output itself (accumulate)
    res = rnd(6, M, N)
    y2 = empty(ctx, M, N)
    eng.lora_linear(ctx, xt, wt, t, Bt, y2, residual=up(ctx, res))
    assert_close("lora_linear+residual", y2.to_numpy(), want_y + res, atol=1e-3, rtol=1e-4)
    acc = rnd(7, M, K)
    dx2 = up(ctx, acc)
    eng.lora_linear_dx(ctx, dyt, wt, dt, At, dx2, residual=dx2)
    assert_close("lora_linear_dx accumulate", dx2.to_numpy(), want_dx + acc, atol=2e-3, rtol=1e-4)
    db, da = empty(ctx, r, N), empty(ctx, K, r)
    eng.lora_grad_b(ctx, t, dyt, db)
    eng.lora_grad_a(ctx, xt, dt, da)
    assert_close("dB", db.to_numpy(), grads["l.lora_b"], atol=2e-3, rtol=1e-4)
    assert_close("dA", da.to_numpy(), grads["l.lora_a"], atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("M,K,Ns,r,f16", [(256, 960, (960, 320, 320), 8, True), (100, 64, (64, 32, 96), 4, True),
                                          (192, 128, (320, 256), 0, True), (64, 32, (48, 40), 8, False),
                                          (130, 96, (40, 72, 8), 16, True),
                                          # the step's own shapes: the summed input gradient runs its K segments on eight waves
                                          (2048, 960, (960, 320, 320), 8, True), (2048, 960, (2560, 2560), 0, True)])
def test_grouped_linears_match_single_calls(g, M, K, Ns, r, f16):
    """q/k/v (gate/up) of one input in one launch, and their summed input gradient in one launch."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    x = rnd(1, M, K)
    xt = up(ctx, x)
    fwd, bwd, want_dx = [], [], np.zeros((M, K), np.float32)
    res = rnd(50, M, K)
    for i, N in enumerate(Ns):
        w = rnd(10 + i, K, N, scale=0.05)
        wr = cpu.round_f16(w) if f16 else w
        wt = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N]) if f16 else up(ctx, w)
        dy = rnd(20 + i, M, N)
        if r:
            A, B = rnd(30 + i, K, r, scale=0.1), rnd(40 + i, r, N, scale=0.1)
            t, dt = rnd(60 + i, M, r), rnd(70 + i, M, r)
            want_y = cpu.matmul(x, wr) + cpu.matmul(t, B)
            want_dx += cpu.matmul(dy, np.ascontiguousarray(wr.T)) + cpu.matmul(dt, np.ascontiguousarray(A.T))
            y = empty(ctx, M, N)
            fwd.append((wt, up(ctx, t), up(ctx, B), y, None))
            bwd.append((up(ctx, dy), wt, up(ctx, dt), up(ctx, A)))
        else:
            want_y = cpu.matmul(x, wr)
            want_dx += cpu.matmul(dy, np.ascontiguousarray(wr.T))
            y = empty(ctx, M, N)
            fwd.append((wt, None, None, y, None))
            bwd.append((up(ctx, dy), wt, None, None))
        fwd[-1] = fwd[-1] + (want_y,)
    eng.lora_linear_group(ctx, xt, [f[:5] for f in fwd])
    for i, f in enumerate(fwd):
        assert_close("group y%d" % i, f[3].to_numpy(), f[5], atol=1e-3, rtol=1e-4)
    dx = empty(ctx, M, K)
    eng.lora_linear_dx_group(ctx, bwd, dx)
    # the reference's GEMM bar for N(0,1) operands is 1e-3 + 1e-4*|want| per product (gpu_kernels.rs:1072-1077);
    # dx is the sum of len(Ns) such products (one per grouped linear), each with its own rounding: 3e-3
    assert_close("group dx", dx.to_numpy(), want_dx, atol=3e-3, rtol=1e-4)
    dx2 = up(ctx, res)
    eng.lora_linear_dx_group(ctx, bwd, dx2, residual=dx2)
    assert_close("group dx + residual", dx2.to_numpy(), want_dx + res, atol=3e-3, rtol=1e-4)


@pytest.mark.parametrize("B,S,K,heads,kv,r,f16", [(2, 64, 192, 3, 1, 8, True), (1, 32, 64, 2, 2, 0, True),
                                                  (2, 24, 96, 2, 1, 4, False)])
def test_grouped_projections_with_rope_in_the_epilogue(g, B, S, K, heads, kv, r, f16):
    """q and k rotated inside the projection launch (heads of 64) == projection followed by rope."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    D, M, theta = 64, B * S, 10000.0
    x = rnd(1, M, K)
    table = eng.rope_table(ctx, S, D, 0, theta)
    items, wants = [], []
    for i, N in enumerate((heads * D, kv * D, kv * D)):
        w = rnd(10 + i, K, N, scale=0.05)
        wr = cpu.round_f16(w) if f16 else w
        wt = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N]) if f16 else up(ctx, w)
        want = cpu.matmul(x, wr)
        t = bm = None
        if r:
            tt, bb = rnd(20 + i, M, r), rnd(30 + i, r, N, scale=0.1)
            want = want + cpu.matmul(tt, bb)
            t, bm = up(ctx, tt), up(ctx, bb)
        if i < 2:
            want = cpu.rope(want.reshape(B, S, N), D, 0, theta).reshape(M, N)
        items.append((wt, t, bm, empty(ctx, M, N), None))
        wants.append(want)
    eng.lora_linear_group(ctx, up(ctx, x), items, rope_table=table, rope_seq=S, n_rope=2)
    for i, (it, want) in enumerate(zip(items, wants)):
        assert_close("rotated projection %d" % i, it[3].to_numpy(), want, atol=1e-3, rtol=1e-4)
    # the table-driven rotation on its own, both directions
    y = rnd(40, B, S, heads * D)
    out = empty(ctx, B, S, heads * D)
    eng.rope_apply(ctx, up(ctx, y.reshape(B, S, heads * D)), out, D, table)
    assert_close("rope_apply", out.to_numpy().reshape(y.shape), cpu.rope(y, D, 0, theta))
    back = empty(ctx, B, S, heads * D)
    eng.rope_apply(ctx, out, back, D, table, inverse=True)
    assert_close("rope_apply inverse", back.to_numpy().reshape(y.shape), y, atol=1e-5)


@pytest.mark.parametrize("M,H,F,f16", [(256, 960, 2560, True), (100, 64, 96, True), (70, 32, 40, True),
                                       (64, 32, 48, False)])
def test_fused_gated_mlp_halves(g, M, H, F, f16):
    """gate/up projections + silu_gate in one launch; down-projection backward + silu_gate backward in one."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    x = rnd(1, M, H)
    wg, wu, wd = rnd(2, H, F, scale=0.1), rnd(3, H, F, scale=0.1), rnd(4, F, H, scale=0.1)
    rd = (lambda w: cpu.round_f16(w)) if f16 else (lambda w: w)
    mk = (lambda w: UnifiedTensor.from_f32_as_f16(ctx, w, list(w.shape))) if f16 else (lambda w: up(ctx, w))
    want_gate, want_up = cpu.matmul(x, rd(wg)), cpu.matmul(x, rd(wu))
    want_act = cpu.silu_gate(want_gate, want_up)
    gate, upt, act = empty(ctx, M, F), empty(ctx, M, F), empty(ctx, M, F)
    eng.mlp_gate_up(ctx, up(ctx, x), mk(wg), mk(wu), gate, upt, act)
    assert_close("gate", gate.to_numpy(), want_gate, atol=1e-3, rtol=1e-4)
    assert_close("up", upt.to_numpy(), want_up, atol=1e-3, rtol=1e-4)
    assert_close("act", act.to_numpy(), want_act, atol=1e-3, rtol=1e-3)

    dy = rnd(5, M, H)
    gate_in, up_in = rnd(6, M, F), rnd(7, M, F)
    d_act = cpu.matmul(dy, np.ascontiguousarray(rd(wd).T))
    want_dg, want_du = cpu.silu_gate_backward(gate_in, up_in, d_act)
    d_gate, d_up, scratch = empty(ctx, M, F), empty(ctx, M, F), empty(ctx, M, F)
    eng.mlp_down_backward(ctx, up(ctx, dy), mk(wd), up(ctx, gate_in), up(ctx, up_in), d_gate, d_up, scratch)
    # d_act = dy @ W_down^T is a GEMM of N(0,1) operands (the reference's bar: 1e-3 + 1e-4*|d_act|); the
    # SiLU-gate backward multiplies it by up * silu'(gate) resp. silu(gate), factors of N(0,1) inputs that
    # exceed 1 in magnitude for a third of the elements and reach 3-4: twice the GEMM's absolute term
    assert_close("d_gate", d_gate.to_numpy(), want_dg, atol=2e-3, rtol=1e-3)
    assert_close("d_up", d_up.to_numpy(), want_du, atol=2e-3, rtol=1e-3)


@pytest.mark.parametrize("rows,size", [(1, 1), (3, 7), (37, 96), (16, 576), (64, 960), (5, 2048), (3, 2100),
                                       (2048, 576), (4100, 960), (2500, 1536)])
def test_rms_norm_forward_backward(g, rows, size):
    ctx, eng = g
    x, w, gy = rnd(1, rows, size), rnd(2, size), rnd(3, rows, size)
    eps = 1e-5
    out = empty(ctx, rows, size)
    eng.rms_norm_eps(ctx, up(ctx, x), up(ctx, w), out, eps)
    assert_close("rms_norm", out.to_numpy(), cpu.rms_norm(x, w, eps))
    gx, gw = empty(ctx, rows, size), empty(ctx, size)
    eng.rms_norm_backward(ctx, up(ctx, x), up(ctx, w), up(ctx, gy), gx, gw, eps)
    want_gx, want_gw = cpu.rms_norm_backward(x, w, gy, eps)
    assert_close("rms gx", gx.to_numpy(), want_gx)
    # gw sums g*x*inv over the rows: up to 4100 terms of magnitude ~1 (|gw| ~ sqrt(rows) = 64), added in
    # f32 in another order than the oracle's: the absolute term is doubled for the elements near zero
    assert_close("rms gw", gw.to_numpy(), want_gw, atol=2e-4)
    gx2 = empty(ctx, rows, size)
    eng.rms_norm_backward(ctx, up(ctx, x), up(ctx, w), up(ctx, gy), gx2, None, eps)
    assert_close("rms gx (no gw)", gx2.to_numpy(), want_gx)


@pytest.mark.parametrize("B,S,heads,D,pos,theta", [(1, 1, 1, 2, 0, 10000.0), (2, 9, 3, 8, 5, 10000.0),
                                                  (2, 256, 9, 64, 0, 100000.0), (1, 64, 4, 64, 960, 500.0)])
def test_rope_forward_and_inverse(g, B, S, heads, D, pos, theta):
    ctx, eng = g
    x = rnd(11, B, S, heads * D)
    t = up(ctx, x)
    eng.rope_theta(ctx, t, D, pos, theta)
    want = cpu.rope(x, D, pos, theta)
    assert_close("rope", t.to_numpy(), want)
    eng.rope_theta_inverse(ctx, t, D, pos, theta)
    assert_close("rope inverse", t.to_numpy(), x)


@pytest.mark.parametrize("n", [1, 5, 64, 1000, 4096 * 3 + 1])
def test_elementwise(g, n):
    ctx, eng = g
    a, b, gy = rnd(1, n, scale=3.0), rnd(2, n), rnd(3, n)
    out = empty(ctx, n)
    eng.add(ctx, up(ctx, a), up(ctx, b), out)
    np.testing.assert_array_equal(out.to_numpy(), a + b)
    ga, gb = empty(ctx, n), empty(ctx, n)
    eng.add_backward(ctx, up(ctx, gy), ga, gb)
    np.testing.assert_array_equal(ga.to_numpy(), gy)
    np.testing.assert_array_equal(gb.to_numpy(), gy)
    eng.silu_gate_fused(ctx, up(ctx, a), up(ctx, b), out)
    assert_close("silu_gate", out.to_numpy(), cpu.silu_gate(a, b))
    eng.silu_gate_backward(ctx, up(ctx, a), up(ctx, b), up(ctx, gy), ga, gb)
    wa, wb = cpu.silu_gate_backward(a, b, gy)
    assert_close("silu ga", ga.to_numpy(), wa)
    assert_close("silu gb", gb.to_numpy(), wb)
    t = up(ctx, a)
    eng.gradient_scale(ctx, t, 0.37)
    np.testing.assert_array_equal(t.to_numpy(), a * np.float32(0.37))
    eng.gradient_accumulate(ctx, t, up(ctx, b))
    np.testing.assert_array_equal(t.to_numpy(), a * np.float32(0.37) + b)


@pytest.mark.parametrize("n", [1, 7, 4096 + 3, 1 << 20])
def test_clip_grad_by_norm_scales_in_place(g, n):
    """`clip_grad_by_norm` (engine/training.rs:161-169, WGSL grad_clip): x *= scale, one f32 product per
    element, so bit-exact against numpy; together with `sum_squares_partial` it is the reference's clip."""
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    x = rnd(n, n, scale=3.0)
    parts = UnifiedTensor.zeros(ctx, [(n + 4095) // 4096])
    t = up(ctx, x)
    assert eng.sum_squares_partial(ctx, t, parts, 0) == (n + 4095) // 4096
    norm = np.float32(np.sqrt(parts.to_numpy().astype(np.float64).sum()))
    assert abs(float(norm) - float(rs.global_grad_norm([x]))) <= 1e-5 * float(norm)
    scale = np.float32(1.0) / (norm + np.float32(1e-6))
    eng.clip_grad_by_norm(ctx, t, float(scale))
    np.testing.assert_array_equal(t.to_numpy(), cpu.scale(x, float(scale)))
    np.testing.assert_array_equal(t.to_numpy(), x * scale)


def test_copy_tensor_with_a_destination_offset(g):
    """`copy_tensor(src, dst, dst_byte_offset)` (engine/mod.rs:399-415): device to device, bytes outside the
    written range untouched; f16 buffers copy as raw bytes."""
    from ferrotensor_amd import FtError, UnifiedTensor
    ctx, eng = g
    base, src = rnd(1, 1000), rnd(2, 300)
    dst = up(ctx, base)
    eng.copy_tensor(ctx, up(ctx, src), dst, dst_byte_offset=4 * 123)
    want = base.copy()
    want[123:423] = src
    np.testing.assert_array_equal(dst.to_numpy(), want)
    eng.copy_tensor(ctx, up(ctx, src), dst)
    want[:300] = src
    np.testing.assert_array_equal(dst.to_numpy(), want)
    h = UnifiedTensor.from_f32_as_f16(ctx, src, [300])
    d16 = UnifiedTensor.from_f32_as_f16(ctx, base, [1000])
    eng.copy_tensor(ctx, h, d16, dst_byte_offset=2 * 400)
    want16 = cpu.pack_f16(base)
    want16[400:700] = cpu.pack_f16(src)
    np.testing.assert_array_equal(d16.to_vec(ctx, np.uint16), want16)


@pytest.mark.parametrize("B,S,heads,D,pos,theta", [(2, 9, 3, 8, 5, 10000.0), (2, 64, 5, 64, 0, 100000.0),
                                                  (1, 33, 2, 6, 960, 500.0)])
def test_rope_theta_out_of_place(g, B, S, heads, D, pos, theta):
    """`ft_rope_theta_to`: the rotation written to a second buffer (what `Tensor::rope_theta` and
    `RoPENode::backward` get by copying first, autograd/src/lib.rs:509-533, 1122-1139); the source keeps its bits
    and both directions equal the in-place kernels bit for bit."""
    ctx, eng = g
    x = rnd(12, B, S, heads * D)
    src, dst = up(ctx, x), empty(ctx, B, S, heads * D)
    eng.rope_theta_to(ctx, src, dst, D, pos, theta)
    np.testing.assert_array_equal(src.to_numpy(), x)
    assert_close("rope_to", dst.to_numpy(), cpu.rope(x, D, pos, theta))
    inplace = up(ctx, x)
    eng.rope_theta(ctx, inplace, D, pos, theta)
    np.testing.assert_array_equal(dst.to_numpy(), inplace.to_numpy())
    back = empty(ctx, B, S, heads * D)
    eng.rope_theta_to(ctx, dst, back, D, pos, theta, inverse=True)
    assert_close("rope_to inverse", back.to_numpy(), x)
    assert_close("rope_to inverse vs oracle", back.to_numpy(), cpu.rope(dst.to_numpy(), D, pos, theta, inverse=True))
    eng.rope_theta_inverse(ctx, inplace, D, pos, theta)
    np.testing.assert_array_equal(back.to_numpy(), inplace.to_numpy())


def test_pool_reuses_exact_sizes_and_trims(g):
    """The buffer pool (`pool.rs`): a freed buffer serves the next request of exactly its size; `ft_pool_trim`
    hands the idle ones back to the device."""
    ctx, _ = g
    ctx.synchronize()
    ctx.pool_trim()
    live0, idle0 = ctx.pool_stats()
    assert idle0 == 0
    n, n2 = 12800, 12864                 # 51200 and 51456 bytes: two size classes (256-byte granularity)
    a = empty(ctx, n)
    ptr = a.ptr
    live1, _ = ctx.pool_stats()
    assert live1 == live0 + n * 4
    del a
    live2, idle2 = ctx.pool_stats()
    assert live2 == live0 and idle2 == n * 4
    b = empty(ctx, n)
    assert b.ptr == ptr and ctx.pool_stats()[1] == 0
    c = empty(ctx, n2)
    assert c.ptr != ptr
    del b, c
    assert ctx.pool_stats()[1] == n * 4 + n2 * 4
    ctx.pool_trim()
    assert ctx.pool_stats() == (live0, 0)


def test_embedding_gather_bit_exact(g):
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    table = rnd(5, 50, 24)
    ids = np.array([0, 49, 7, 50, 4000000000, 3], np.uint32)
    out = empty(ctx, ids.size, 24)
    eng.embedding(ctx, up(ctx, table), UnifiedTensor.from_bytes(ctx, ids, [ids.size]), out)
    np.testing.assert_array_equal(out.to_numpy(), cpu.embedding(table, ids))


@pytest.mark.parametrize("rows,vocab", [(4, 7), (8, 32), (12, 50), (9, 4096), (5, 16384 + 4), (3, 49152), (2, 50000)])
def test_masked_cross_entropy(g, rows, vocab):
    from ferrotensor_amd import UnifiedTensor
    ctx, eng = g
    rng = np.random.default_rng(rows * vocab)
    logits = rnd(3, rows, vocab, scale=4.0)
    targets = rng.integers(0, vocab, rows).astype(np.uint32)
    targets[rows // 2] = rs.MASKED_CE_SKIP
    weights = rng.random(rows).astype(np.float32)
    want_g, want_l = cpu.masked_cross_entropy(logits, targets, weights)
    grad, row_loss = empty(ctx, rows, vocab), empty(ctx, rows)
    tl = up(ctx, logits)
    tt = UnifiedTensor.from_bytes(ctx, targets, [rows])
    eng.masked_cross_entropy_weighted(ctx, tl, tt, up(ctx, weights), grad, row_loss)
    assert_close("ce loss", row_loss.to_numpy(), want_l)
    assert_close("ce grad", grad.to_numpy(), want_g, atol=1e-6)
    skipped = targets == rs.MASKED_CE_SKIP
    assert (grad.to_numpy()[skipped] == 0).all() and (row_loss.to_numpy()[skipped] == 0).all()
    # in place, with the upstream scale folded in
    eng.masked_cross_entropy_weighted(ctx, tl, tt, up(ctx, weights), tl, row_loss, grad_scale=0.125)
    assert_close("ce grad in place", tl.to_numpy(), want_g * np.float32(0.125), atol=1e-6)
    assert_close("ce loss in place", row_loss.to_numpy(), want_l)


def test_sum_squares_and_adamw(g):
    ctx, eng = g
    from ferrotensor_amd import AdamParams, UnifiedTensor
    x = rnd(9, 4096 * 2 + 100)
    out = UnifiedTensor.zeros(ctx, [8])
    n = eng.sum_squares_partial(ctx, up(ctx, x), out, 3)
    want = np.zeros(8, np.float32)
    assert n == cpu.sum_squares_partial(x, want, 3) == 3
    assert_close("sum squares", out.to_numpy(), want, atol=1e-3)

    n = 4096 * 5 + 17
    w0, gr = rnd(1, n), rnd(2, n)
    m0, v0 = rnd(3, n, scale=0.1), np.abs(rnd(4, n, scale=0.1))
    for wd, t in [(0.0, 1.0), (0.01, 7.0)]:
        p = AdamParams(lr=1e-3, weight_decay=wd, t=t)
        w, m, v = w0.copy(), m0.copy(), v0.copy()
        cpu.adamw_update(w, gr, m, v, p.lr, p.beta1, p.beta2, p.eps, p.weight_decay, p.t)
        tw, tm, tv = up(ctx, w0), up(ctx, m0), up(ctx, v0)
        eng.adamw_update(ctx, tw, up(ctx, gr), tm, tv, p)
        assert_close("adamw w", tw.to_numpy(), w, atol=1e-6, rtol=1e-5)
        assert_close("adamw m", tm.to_numpy(), m, atol=1e-7, rtol=1e-5)
        assert_close("adamw v", tv.to_numpy(), v, atol=1e-7, rtol=1e-5)
        # multi-tensor launch over uneven pieces gives the same numbers
        cuts = [0, 100, 4096 + 100, n]
        parts = lambda a: [up(ctx, a[cuts[i]:cuts[i + 1]]) for i in range(3)]
        ws, gs, ms, vs = parts(w0), parts(gr), parts(m0), parts(v0)
        eng.adamw_update_multi(ctx, ws, gs, ms, vs, p)
        got = np.concatenate([t_.to_numpy() for t_ in ws])
        np.testing.assert_array_equal(got, tw.to_numpy())


def test_adamw_four_million_parameters(g):
    """The kernel-microbench AdamW case: one fused update over 4M f32 parameters."""
    ctx, eng = g
    from ferrotensor_amd import AdamParams
    n = 4 * 1024 * 1024
    w0, gr = rnd(1, n), rnd(2, n)
    m0, v0 = rnd(3, n, scale=0.1), np.abs(rnd(4, n, scale=0.1))
    p = AdamParams(lr=2e-4, weight_decay=0.01, t=3.0)
    w, m, v = w0.copy(), m0.copy(), v0.copy()
    cpu.adamw_update(w, gr, m, v, p.lr, p.beta1, p.beta2, p.eps, p.weight_decay, p.t)
    tw, tm, tv = up(ctx, w0), up(ctx, m0), up(ctx, v0)
    eng.adamw_update(ctx, tw, up(ctx, gr), tm, tv, p)
    assert_close("adamw w", tw.to_numpy(), w, atol=1e-6, rtol=1e-5)
    assert_close("adamw m", tm.to_numpy(), m, atol=1e-7, rtol=1e-5)
    assert_close("adamw v", tv.to_numpy(), v, atol=1e-7, rtol=1e-5)


def test_mfma_probe_reports_time_and_flops(g):
    """The matrix-pipe probe runs the stated number of MFMAs (4096 flop each) and its rate stays under the peak."""
    from ferrotensor_amd import FtError
    ctx, _ = g
    seconds, flops = ctx.mfma_probe(200, waves_per_simd=2, chains=4)
    waves = 256 * 2 * 4
    assert flops == waves * 200 * 16 * 4096.0
    assert seconds > 0 and flops / seconds < 157.3e12 * 1.02
    s1, _ = ctx.mfma_probe(200, waves_per_simd=1, chains=1, random_operands=False)
    assert s1 > 0
    with pytest.raises(FtError):
        ctx.mfma_probe(10, waves_per_simd=9)
    with pytest.raises(FtError):
        ctx.mfma_probe(10, chains=3)


def test_errors_are_reported_not_fatal(g):
    from ferrotensor_amd import FtError
    ctx, eng = g
    x = up(ctx, rnd(1, 4, 6))
    with pytest.raises(FtError):
        eng.rope_theta(ctx, x, 4, 0, 10000.0)  # hidden 6 is not a multiple of head_dim 4
    with pytest.raises(FtError):
        eng.lora_down(ctx, x, up(ctx, rnd(2, 6, 40)), empty(ctx, 4, 40), 1.0)  # rank > 32


# ---- attention (gpu_kernels.rs cpu_attention :132-179, cpu_attention_backward :183-224) ----

ATTN_CASES = [
    # B, Sq, Sk, H, Hkv, D, causal, offset
    (1, 1, 1, 1, 1, 8, True, 0),
    (2, 16, 16, 4, 2, 8, True, 0),          # tiny config of the gradient fixture
    (2, 13, 13, 4, 2, 8, True, 0),
    (1, 40, 40, 6, 6, 16, True, 0),
    (2, 17, 17, 3, 1, 64, False, 0),
    (1, 100, 100, 2, 2, 64, True, 0),
    (2, 256, 256, 9, 3, 64, True, 0),       # SmolLM2-135M heads at seq 256
    (8, 256, 256, 9, 3, 64, True, 0),       # the kernel-microbench attention case, full size
    (2, 256, 256, 15, 5, 64, True, 0),      # SmolLM2-360M heads
    (1, 256, 256, 15, 5, 64, True, 0),      # one sequence per pass: dK/dV per query head + ordered sum, dQ on 4 waves
    (1, 1024, 1024, 32, 32, 64, True, 0),   # SmolLM2-1.7B heads at seq 1024 (no grouping)
    (2, 1024, 1024, 8, 2, 64, True, 0),     # grouped heads at seq 1024
    (1, 70, 70, 2, 1, 128, True, 0),
    (1, 33, 65, 2, 1, 32, True, 32),        # queries at positions 32.. against a longer key run
    (1, 5, 37, 4, 4, 24, False, 0),
    # the 16-row kernels (head_dim 64): the headline batch (64-row tiles, 16 waves), half of it (32-row tiles),
    # ragged lengths, queries offset against a longer key run, no mask
    (8, 256, 256, 15, 5, 64, True, 0),
    (4, 256, 256, 15, 5, 64, True, 0),
    (3, 70, 70, 4, 2, 64, True, 0),
    (1, 33, 65, 2, 1, 64, True, 32),
    (40, 50, 50, 4, 2, 64, True, 3),
    (2, 130, 200, 4, 4, 64, False, 0),
]


@pytest.mark.parametrize("B,Sq,Sk,H,Hkv,D,causal,offset", ATTN_CASES)
def test_flash_attention_forward_backward(g, B, Sq, Sk, H, Hkv, D, causal, offset):
    from ferrotensor_amd import AttentionOptions, UnifiedTensor
    ctx, eng = g
    # operands uniform in [-1, 1) as the reference's attention tests draw them (rand_vec,
    # gpu_kernels.rs:36-48), so its bar for dq / dk / dv applies unchanged (gpu_kernels.rs:1929-1931)
    uni = lambda seed, *shape: np.random.default_rng(seed).uniform(-1.0, 1.0, shape).astype(np.float32)
    q, k, v = uni(1, B, Sq, H, D), uni(2, B, Sk, Hkv, D), uni(3, B, Sk, Hkv, D)
    do = uni(4, B, Sq, H, D)
    want_o, want_lse = cpu.attention(q, k, v, causal=causal, causal_offset=offset)
    want_dq, want_dk, want_dv = cpu.attention_backward(q, k, v, want_o, do, causal=causal, causal_offset=offset)
    opts = AttentionOptions(causal=causal, causal_offset=offset)
    tq, tk, tv, tdo = up(ctx, q), up(ctx, k), up(ctx, v), up(ctx, do)
    out = empty(ctx, B, Sq, H, D)
    stats = UnifiedTensor.zeros(ctx, [B, H, Sq, 2])
    eng.flash_attention_v2_with_stats(ctx, tq, tk, tv, out, stats, opts)
    assert_close("attention out", out.to_numpy(), want_o)
    assert_close("attention lse", stats.to_numpy()[..., 1], want_lse)
    dq, dk, dv = empty(ctx, B, Sq, H, D), empty(ctx, B, Sk, Hkv, D), empty(ctx, B, Sk, Hkv, D)
    eng.flash_attention_v2_backward_with_stats(ctx, tq, tk, tv, out, tdo, dq, dk, dv, stats, opts)
    delta = (do.astype(np.float64) * want_o.astype(np.float64)).sum(-1).transpose(0, 2, 1)
    assert_close("attention delta", stats.to_numpy()[..., 0], delta)
    assert_close("dq", dq.to_numpy(), want_dq)
    assert_close("dk", dk.to_numpy(), want_dk)
    assert_close("dv", dv.to_numpy(), want_dv)
    # forward without stats gives the same output
    out2 = empty(ctx, B, Sq, H, D)
    eng.flash_attention_v2_with(ctx, tq, tk, tv, out2, opts)
    np.testing.assert_array_equal(out2.to_numpy(), out.to_numpy())


def test_attention_causality_is_bit_exact(g):
    """Changing later tokens leaves earlier outputs untouched (model_correctness.rs:281-300)."""
    from ferrotensor_amd import AttentionOptions
    ctx, eng = g
    q, k, v = rnd(1, 1, 96, 3, 64), rnd(2, 1, 96, 1, 64), rnd(3, 1, 96, 1, 64)
    opts = AttentionOptions(causal=True)
    a = empty(ctx, 1, 96, 3, 64)
    eng.flash_attention_v2_with(ctx, up(ctx, q), up(ctx, k), up(ctx, v), a, opts)
    k2, v2 = k.copy(), v.copy()
    k2[:, 64:], v2[:, 64:] = rnd(5, 1, 32, 1, 64), rnd(6, 1, 32, 1, 64)
    b = empty(ctx, 1, 96, 3, 64)
    eng.flash_attention_v2_with(ctx, up(ctx, q), up(ctx, k2), up(ctx, v2), b, opts)
    np.testing.assert_array_equal(a.to_numpy()[:, :64], b.to_numpy()[:, :64])


def test_attention_rejects_unsupported_options(g):
    from ferrotensor_amd import AttentionOptions, FtError
    ctx, eng = g
    q = up(ctx, rnd(1, 1, 4, 2, 8))
    k = up(ctx, rnd(2, 1, 4, 1, 8))
    out = empty(ctx, 1, 4, 2, 8)
    with pytest.raises(FtError):
        eng.flash_attention_v2_with(ctx, q, k, k, out, AttentionOptions(causal=True, window=2))
    with pytest.raises(FtError):
        eng.flash_attention_v2_with(ctx, q, k, k, out, AttentionOptions(causal=True, dropout_prob=0.1))


def test_unaligned_residual_and_gradient_pointers_take_the_guarded_kernels(g):
    """A residual, or attention gradient buffers, that are 4-byte but not 16-byte aligned (a view into the
    middle of a buffer) must not reach the kernels that use 16-byte accesses: same results as aligned ones."""
    import ctypes as C
    from ferrotensor_amd import AttentionOptions, UnifiedTensor
    from ferrotensor_amd._lib import check
    ctx, eng = g
    lib = ctx._lib
    M, K, N = 256, 128, 192
    x, w, res = rnd(1, M, K), rnd(2, K, N, scale=0.05), rnd(3, M * N + 1)
    wt = UnifiedTensor.from_f32_as_f16(ctx, w, [K, N])
    xt, rest, y = up(ctx, x), up(ctx, res), empty(ctx, M, N)
    off = C.c_void_p(rest.ptr + 4)                       # element 1 of the residual buffer
    check(lib.ft_lora_linear(ctx.handle, C.c_void_p(xt.ptr), C.c_void_p(wt.ptr), wt.dtype, None, None, off,
                             C.c_void_p(y.ptr), M, K, N, 0))
    want = f64_mm(x, cpu.round_f16(w)) + res[1:].reshape(M, N)
    assert_close("residual at an odd offset", y.to_numpy(), want, atol=1e-3, rtol=1e-4)

    B, S, H, D = 1, 64, 2, 64
    q, k, v, do = rnd(4, B, S, H, D), rnd(5, B, S, H, D), rnd(6, B, S, H, D), rnd(7, B, S, H, D)
    opts = AttentionOptions(causal=True)
    tq, tk, tv, tdo = up(ctx, q), up(ctx, k), up(ctx, v), up(ctx, do)
    out, stats = empty(ctx, B, S, H, D), UnifiedTensor.zeros(ctx, [B, H, S, 2])
    eng.flash_attention_v2_with_stats(ctx, tq, tk, tv, out, stats, opts)
    dq, dk, dv = empty(ctx, B, S, H, D), empty(ctx, B, S, H, D), empty(ctx, B, S, H, D)
    eng.flash_attention_v2_backward_with_stats(ctx, tq, tk, tv, out, tdo, dq, dk, dv, stats, opts)
    n = B * S * H * D
    odd = [UnifiedTensor.zeros(ctx, [n + 1]) for _ in range(3)]
    o = opts.c()
    check(lib.ft_flash_attention_v2_backward_with_stats(
        ctx.handle, C.c_void_p(tq.ptr), C.c_void_p(tk.ptr), C.c_void_p(tv.ptr), C.c_void_p(out.ptr),
        C.c_void_p(tdo.ptr), C.c_void_p(odd[0].ptr + 4), C.c_void_p(odd[1].ptr + 4), C.c_void_p(odd[2].ptr + 4),
        C.c_void_p(stats.ptr), B, S, S, H, H, D, C.byref(o)))
    for name, a, b in (("dq", dq, odd[0]), ("dk", dk, odd[1]), ("dv", dv, odd[2])):
        got = b.to_numpy()
        assert got[0] == 0.0
        assert_close(name + " at an odd offset", got[1:], a.to_numpy().reshape(-1), atol=2e-5)
