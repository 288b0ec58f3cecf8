"""Parity of every HIP kernel (through the C ABI) with the CPU oracle.

Integer stages (codes, int32 accumulators) must be bit-exact; step sizes are
fp32 values computed by the same IEEE operations and must be equal too.
"""
import numpy as np
import pytest
import torch

from oracle import hot_oracle as orc

pytestmark = pytest.mark.gpu

TDT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def make_input(M, K, dtype, seed, outliers=True):
    """g_y-like data: N(0, 1e-3) with 1 % of entries x50, rounded to dtype."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g) * 1e-3
    if outliers:
        mask = torch.rand(M, K, generator=g) < 0.01
        x = torch.where(mask, x * 50, x)
    x = x.to(TDT[dtype])
    return x, x.float().numpy()


def np_codes(codes, bits, K):
    c = codes.cpu().numpy()
    return orc.unpack_int4(c)[:, :K] if bits == 4 else c[:, :K]


# ---------------------------------------------------------------- hq_rowwise

@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("n", [16, 32, 64])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("scale", ["tensor", "row"])
def test_hq_rowwise_nearest(gpu, dtype, n, bits, scale):
    from hot_amd import ops
    M, K = 300, 768
    x, xn = make_input(M, K, dtype, seed=n + bits)
    codes, s = ops.hq_rowwise(x.to(gpu), n=n, bits=bits, rounding="nearest", scale=scale)
    mode = orc.SCALE_ROW if scale == "row" else orc.SCALE_TENSOR
    q_ref, s_ref = orc.quant(orc.fwht_blocks_last(xn, n), bits, mode)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(np_codes(codes, bits, K), q_ref)


@pytest.mark.parametrize("K", [16, 64, 1024, 3072, 4096, 11008, 20480])
@pytest.mark.parametrize("scale", ["tensor", "row"])
def test_hq_rowwise_widths(gpu, K, scale):
    """Every per-row chunk count the dispatcher can pick, and ragged last sweeps."""
    from hot_amd import ops
    M = 37
    x, xn = make_input(M, K, "bf16", seed=K)
    codes, s = ops.hq_rowwise(x.to(gpu), n=16, bits=4, scale=scale)
    mode = orc.SCALE_ROW if scale == "row" else orc.SCALE_TENSOR
    q_ref, s_ref = orc.quant(orc.fwht_blocks_last(xn, 16), 4, mode)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(np_codes(codes, 4, K), q_ref)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("scale", ["tensor", "row"])
def test_hq_rowwise_stochastic_matches_oracle(gpu, dtype, bits, scale):
    """Same counter-based RNG on both sides: identical codes for a given seed."""
    from hot_amd import ops
    M, K = 200, 1536
    x, xn = make_input(M, K, dtype, seed=5)
    seed = 0x1234_5678_9ABC_DEF0
    codes, s = ops.hq_rowwise(x.to(gpu), n=16, bits=bits, rounding="stoch", scale=scale, seed=seed)
    mode = orc.SCALE_ROW if scale == "row" else orc.SCALE_TENSOR
    q_ref, s_ref = orc.quant(orc.fwht_blocks_last(xn, 16), bits, mode, orc.ROUND_STOCH, seed, orc.STREAM_GX)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(np_codes(codes, bits, K), q_ref)


def test_hq_rowwise_stochastic_unbiased(gpu):
    """E[q] = y over seeds: the mean code of many seeds approaches y = t/d and
    every code is floor(y) or ceil(y)."""
    from hot_amd import ops
    M, K = 64, 256
    x, xn = make_input(M, K, "f32", seed=11, outliers=False)
    t = orc.fwht_blocks_last(xn, 16)
    s, _ = orc.quant_scale(t, 4, orc.SCALE_TENSOR)
    y = t / (s + np.float32(orc.EPS))
    xd = x.to(gpu)
    nseed = 400
    acc = np.zeros_like(y, dtype=np.float64)
    for seed in range(nseed):
        codes, _ = ops.hq_rowwise(xd, n=16, bits=4, rounding="stoch", scale="tensor", seed=seed)
        q = np_codes(codes, 4, K).astype(np.float64)
        assert np.all((q == np.floor(y)) | (q == np.ceil(y)))
        acc += q
    err = acc / nseed - y
    # per-element std of the mean <= 0.5/sqrt(nseed) = 0.025; allow 5 sigma per element and a tight global mean
    assert np.max(np.abs(err)) < 0.13
    assert abs(err.mean()) < 5 * 0.5 / np.sqrt(nseed * y.size)


def test_hq_rowwise_zero_and_empty(gpu):
    from hot_amd import ops
    z = torch.zeros(8, 64, device=gpu)
    for scale in ("tensor", "row"):
        codes, s = ops.hq_rowwise(z, n=16, bits=4, scale=scale)
        assert torch.all(codes == 0) and torch.all(s == 0)
    e = torch.zeros(0, 64, device=gpu)
    codes, s = ops.hq_rowwise(e, n=16, bits=8, scale="row")
    assert codes.shape == (0, 64)


@pytest.mark.parametrize("n", [1, 2, 4, 8])
@pytest.mark.parametrize("bits,scale,rounding", [(4, "tensor", "nearest"), (8, "row", "nearest"), (4, "row", "stoch")])
def test_hq_rowwise_small_blocks(gpu, n, bits, scale, rounding):
    """Blocks that fit one lane's chunk of 8 elements (heads whose width has few factors of two)."""
    from hot_amd import ops
    M, K = 37, 112
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(n)) * 1e-2
    mode = orc.SCALE_TENSOR if scale == "tensor" else orc.SCALE_ROW
    rnd = orc.ROUND_NEAREST if rounding == "nearest" else orc.ROUND_STOCH
    t = orc.fwht_blocks_last(x.numpy(), n)
    q_ref, s_ref = orc.quant(t, bits, mode, rnd, seed=5, stream=orc.STREAM_GX)
    codes, s = ops.hq_rowwise(x.to(gpu), n=n, bits=bits, scale=scale, rounding=rounding, seed=5)
    got = codes.cpu().numpy()
    full = orc.unpack_int4(got) if bits == 4 else got
    assert np.array_equal(s.cpu().numpy(), np.atleast_1d(s_ref).astype(np.float32).reshape(-1))
    assert np.array_equal(full[:, :K], q_ref)


def test_hq_rowwise_errors(gpu):
    from hot_amd import ops
    from hot_amd._lib import HotError
    with pytest.raises(HotError):
        ops.hq_rowwise(torch.zeros(4, 40, device=gpu), n=16)        # K % n
    with pytest.raises(HotError):
        ops.hq_rowwise(torch.zeros(4, 64, device=gpu), n=12)        # block size: powers of two only
    with pytest.raises(HotError):
        ops.hq_rowwise(torch.zeros(4, 128, device=gpu), n=128)      # ... up to 64
    with pytest.raises(HotError):
        ops.hq_rowwise(torch.zeros(4, 64, device=gpu), bits=5)
    with pytest.raises(RuntimeError):
        ops.hq_rowwise(torch.zeros(4, 64), n=16)                    # not on the GPU
    with pytest.raises(RuntimeError):
        ops.hq_rowwise(torch.zeros(4, 64, 2, device=gpu), n=16)     # not 2-D


# ------------------------------------------------------------------- colwise

def hla_case(L, C, dtype, seed):
    return make_input(L, C, dtype, seed)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("n,rule", [(64, "python"), (16, "paper"), (32, "python"), (1, "python"), (4, "python"), (16, "python")])
@pytest.mark.parametrize("scale", ["tensor", "row"])
def test_hla_tokenwise_nearest(gpu, dtype, n, rule, scale):
    from hot_amd import ops
    L, C = n * 23 if n > 1 else 49, 200
    if rule == "paper":
        _, rows = orc.paper_rows(n, n // 2)
    else:
        nn, rows = orc.hla_rows(n) if n > 1 else (1, np.array([0]))
        assert nn == n
    x, xn = hla_case(L, C, dtype, seed=n)
    codes, s, kout = ops.hla_tokenwise(x.to(gpu), n, list(rows), bits=8, scale=scale)
    t = np.ascontiguousarray(orc.fwht_blocks_first(xn, n, rows).T)  # [C, L']
    assert kout == t.shape[1]
    mode = orc.SCALE_ROW if scale == "row" else orc.SCALE_TENSOR
    q_ref, s_ref = orc.quant(t, 8, mode)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    got = codes.cpu().numpy()
    assert np.array_equal(got[:, :kout], q_ref)
    assert not got[:, kout:].any(), "K padding must be zero"


def test_hla_tokenwise_vit_shape_slice(gpu):
    """n = 64, r = 36 on 12608 tokens (the ViT-B token count), bf16."""
    from hot_amd import ops
    L, C = 12608, 256
    n, rows = orc.hla_rows(L)
    assert (n, len(rows)) == (64, 36)
    x, xn = hla_case(L, C, "bf16", seed=3)
    codes, s, kout = ops.hla_tokenwise(x.to(gpu), n, list(rows), bits=8, scale="tensor")
    assert kout == 7092
    t = np.ascontiguousarray(orc.fwht_blocks_first(xn, n, rows).T)
    q_ref, s_ref = orc.quant(t, 8, orc.SCALE_TENSOR)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    got = codes.cpu().numpy()
    assert np.array_equal(got[:, :kout], q_ref) and not got[:, kout:].any()


@pytest.mark.parametrize("scale", ["tensor", "row"])
def test_hla_tokenwise_stochastic_matches_oracle(gpu, scale):
    from hot_amd import ops
    L, C, n = 64 * 5, 72, 64
    _, rows = orc.hla_rows(64)
    x, xn = hla_case(L, C, "f32", seed=8)
    codes, s, kout = ops.hla_tokenwise(x.to(gpu), n, list(rows), bits=8, rounding="stoch", scale=scale, seed=77)
    t = np.ascontiguousarray(orc.fwht_blocks_first(xn, n, rows).T)
    mode = orc.SCALE_ROW if scale == "row" else orc.SCALE_TENSOR
    q_ref, s_ref = orc.quant(t, 8, mode, orc.ROUND_STOCH, 77, orc.STREAM_GW, index=orc.colwise_rng_index(C, L // n, rows))
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(codes.cpu().numpy()[:, :kout], q_ref)


@pytest.mark.parametrize("scale", ["tensor", "row"])
@pytest.mark.parametrize("L,C,n,rows", [
    (197, 264, 1, [0]),          # one-token blocks: eight consecutive blocks of a channel share a generator call
    (49, 72, 1, [0]),
    (1000, 520, 1, [0]),         # three channel strips, runs of blocks that start off a multiple of eight
    (16 * 21, 40, 16, [5]),      # a single kept row of a 16-token block: numbered the same way
])
def test_hla_tokenwise_stochastic_single_coefficient_blocks(gpu, scale, L, C, n, rows):
    from hot_amd import ops
    x, xn = hla_case(L, C, "f32", seed=L)
    codes, s, kout = ops.hla_tokenwise(x.to(gpu), n, rows, bits=8, rounding="stoch", scale=scale, seed=31)
    t = np.ascontiguousarray(orc.fwht_blocks_first(xn, n, np.asarray(rows)).T)
    mode = orc.SCALE_ROW if scale == "row" else orc.SCALE_TENSOR
    idx = orc.colwise_rng_index(C, L // n, rows)
    assert np.array_equal(idx, np.arange(C * (L // n)).reshape(C, L // n))      # channel * NB + block
    q_ref, s_ref = orc.quant(t, 8, mode, orc.ROUND_STOCH, 31, orc.STREAM_GW, index=idx)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(codes.cpu().numpy()[:, :kout], q_ref)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("n", [16, 32, 64])
def test_wq_colwise_nearest(gpu, dtype, bits, n):
    from hot_amd import ops
    O, I = 64 * 7, 136
    g = torch.Generator().manual_seed(n)
    w = ((torch.rand(O, I, generator=g) * 2 - 1) / np.sqrt(I)).to(TDT[dtype])
    codes, s = ops.wq_colwise(w.to(gpu), n=n, bits=bits)
    t = np.ascontiguousarray(orc.fwht_blocks_first(w.float().numpy(), n).T)  # [I, O]
    q_ref, s_ref = orc.quant(t, bits, orc.SCALE_TENSOR)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    got = codes.cpu().numpy()
    full = orc.unpack_int4(got) if bits == 4 else got
    assert np.array_equal(full[:, :O], q_ref)
    assert not full[:, O:].any()


@pytest.mark.parametrize("bits", [4, 8])
def test_wq_colwise_sawb(gpu, bits):
    from hot_amd import ops
    O, I = 256, 200
    g = torch.Generator().manual_seed(1)
    w = torch.randn(O, I, generator=g) * 0.05
    codes, s = ops.wq_colwise(w.to(gpu), n=16, bits=bits, scale="sawb")
    t = np.ascontiguousarray(orc.fwht_blocks_first(w.numpy(), 16).T)
    q_ref, s_ref = orc.quant(t, bits, orc.SCALE_SAWB)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    got = codes.cpu().numpy()
    full = orc.unpack_int4(got) if bits == 4 else got
    assert np.array_equal(full[:, :O], q_ref)


# ---------------------------------------------------------------------- gemm

def rand_codes(M, K, bits, seed):
    rng = np.random.default_rng(seed)
    qm = 2 ** (bits - 1) - 1
    return rng.integers(-qm, qm + 1, size=(M, K), dtype=np.int8)


def to_operand(q, bits, kp):
    M, K = q.shape
    full = np.zeros((M, kp), dtype=np.int8)
    full[:, :K] = q
    return torch.from_numpy(orc.pack_int4(full) if bits == 4 else full)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (200, 72, 300), (1, 1, 16), (515, 260, 1000), (130, 768, 7092)])
@pytest.mark.parametrize("per_row", [False, True])
def test_gemm_i8_exact(gpu, bits, M, N, K, per_row):
    from hot_amd import ops
    a, b = rand_codes(M, K, bits, 1), rand_codes(N, K, bits, 2)
    kp = ops.kpad(K)
    rng = np.random.default_rng(3)
    sa = rng.uniform(1e-4, 2e-4, size=(M if per_row else 1)).astype(np.float32)
    sb = rng.uniform(1e-3, 2e-3, size=1).astype(np.float32)
    out, acc = ops.gemm_i8(to_operand(a, bits, kp).to(gpu), to_operand(b, bits, kp).to(gpu), K, bits,
                           torch.from_numpy(sa).to(gpu), torch.from_numpy(sb).to(gpu), post_scale=1 / 16,
                           return_acc=True)
    acc_ref = orc.int_gemm_nt(a, b)
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    ref = ((acc_ref.astype(np.float32) * sa.reshape(-1, 1)).astype(np.float32) * sb[0]).astype(np.float32) / np.float32(16)
    assert np.array_equal(out.cpu().numpy(), ref.astype(np.float32))


def test_gemm_i8_extreme_codes(gpu):
    """All operands at +-qmax: the largest accumulators the path can produce."""
    from hot_amd import ops
    for bits, K in ((4, 11008), (8, 7092)):
        qm = 2 ** (bits - 1) - 1
        a = np.full((64, K), qm, dtype=np.int8)
        b = np.full((96, K), -qm, dtype=np.int8)
        kp = ops.kpad(K)
        one = torch.ones(1, device=gpu)
        _, acc = ops.gemm_i8(to_operand(a, bits, kp).to(gpu), to_operand(b, bits, kp).to(gpu), K, bits, one, one,
                             return_acc=True)
        assert torch.all(acc == -qm * qm * K)


def test_gemm_i8_bf16_out(gpu):
    from hot_amd import ops
    a, b = rand_codes(100, 256, 8, 5), rand_codes(60, 256, 8, 6)
    one = torch.ones(1, device=gpu)
    out = ops.gemm_i8(torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu), 256, 8, one, one,
                      out_dtype=torch.bfloat16)
    ref = torch.from_numpy(orc.int_gemm_nt(a, b).astype(np.float32)).to(torch.bfloat16)
    assert torch.equal(out.cpu(), ref)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bits,M,N,K,per_row", [
    (8, 256, 384, 512, False),      # whole tiles: the LDS-staged epilogue
    (4, 384, 256, 1024, True),
    (8, 515, 260, 300, True),       # ragged tiles; 260 columns: four-wide stores, rows not 16-byte aligned in bf16
    (4, 200, 130, 256, False),      # 130 columns: scalar stores
])
def test_gemm_i8_epilogues(gpu, out_dtype, bits, M, N, K, per_row):
    """Every store path of the epilogue, without the int32 side output (which forces the direct one)."""
    from hot_amd import ops
    a, b = rand_codes(M, K, bits, 11), rand_codes(N, K, bits, 12)
    kp = ops.kpad(K)
    rng = np.random.default_rng(13)
    sa = rng.uniform(1e-4, 2e-4, size=(M if per_row else 1)).astype(np.float32)
    sb = rng.uniform(1e-3, 2e-3, size=1).astype(np.float32)
    out = ops.gemm_i8(to_operand(a, bits, kp).to(gpu), to_operand(b, bits, kp).to(gpu), K, bits,
                      torch.from_numpy(sa).to(gpu), torch.from_numpy(sb).to(gpu), post_scale=1 / 64, out_dtype=out_dtype)
    acc = orc.int_gemm_nt(a, b)
    ref = ((acc.astype(np.float32) * sa.reshape(-1, 1)).astype(np.float32) * sb[0]).astype(np.float32) / np.float32(64)
    assert torch.equal(out.cpu(), torch.from_numpy(ref.astype(np.float32)).to(out_dtype))


def exact_acc(a, b):
    """int32 accumulators of A . B^T through BLAS: float32 while every partial sum stays below 2^24
    (then each addition is exact), float64 otherwise."""
    bound = int(np.abs(a).max()) * int(np.abs(b).max()) * a.shape[1]
    dt = np.float32 if bound < 2 ** 24 else np.float64
    return np.rint(a.astype(dt) @ b.astype(dt).T).astype(np.int64).astype(np.int32)


def dequant_ref(acc, sa, sb, post):
    """The epilogue, operation for operation: ((float(acc) * s_a[row]) * s_b) * post."""
    return ((acc.astype(np.float32) * np.asarray(sa, np.float32).reshape(-1, 1)).astype(np.float32)
            * np.float32(sb)).astype(np.float32) * np.float32(post)


# (variant name, bits, M, N, K): shapes ragged on both edges of the variant's own tile, K not a
# multiple of the K tile; the split-K kernel needs fewer than 256 tiles and at least 32 stages.
VARIANT_CASES = [
    ("GEMM_DMA_128_S3", 8, 515, 390, 1000), ("GEMM_DMA_128_S3", 4, 515, 390, 1000),
    ("GEMM_DMA_128_S4", 8, 515, 390, 1000), ("GEMM_DMA_128_S4", 4, 515, 390, 1000),
    ("GEMM_DMA_128_S3", 8, 130, 72, 100), ("GEMM_DMA_128_S4", 4, 1, 1, 16),          # shorter than the ring is deep
    ("GEMM_DMA_256_S4", 8, 700, 530, 600), ("GEMM_DMA_256_S4", 4, 700, 530, 600),
    ("GEMM_DMA_256_S4", 8, 257, 255, 100), ("GEMM_DMA_256_S4", 4, 300, 100, 3000),
    ("GEMM_REG_128", 8, 515, 390, 1000), ("GEMM_REG_128", 4, 515, 390, 1000), ("GEMM_REG_128", 8, 77, 130, 90),
    ("GEMM_DMA_128_SPLITK", 8, 260, 200, 2500), ("GEMM_DMA_128_SPLITK", 4, 260, 200, 5000),
    ("GEMM_DMA_128_SPLITK", 8, 1000, 900, 2100),
    # slot-scheduled kernels: rows of a multiple of 128 bytes (K rounded up to 128 codes, INT4: to 256)
    ("GEMM_SLOT_256", 8, 700, 530, 600), ("GEMM_SLOT_256", 4, 700, 530, 1000), ("GEMM_SLOT_256", 8, 257, 255, 100),
    ("GEMM_SLOT_256", 4, 300, 100, 3000), ("GEMM_SLOT_256", 8, 512, 512, 128),
    ("GEMM_SLOT_128", 8, 515, 390, 1000), ("GEMM_SLOT_128", 4, 515, 390, 1000), ("GEMM_SLOT_128", 8, 130, 72, 100),
    ("GEMM_SLOT_128", 4, 1, 1, 200), ("GEMM_SLOT_128", 8, 384, 256, 7092),
    ("GEMM_SLOT_160X256", 8, 700, 530, 600), ("GEMM_SLOT_160X256", 4, 700, 530, 1000), ("GEMM_SLOT_160X256", 4, 161, 257, 2304),
    ("GEMM_SLOT_160X256", 8, 159, 255, 128), ("GEMM_SLOT_160X256", 4, 1600, 768, 3072),
    # one fragment column per wave: more fragment reads than MFMAs per round (several reads per slot); INT8 only
    ("GEMM_SLOT_96X128", 8, 700, 530, 600), ("GEMM_SLOT_96X128", 8, 97, 129, 128), ("GEMM_SLOT_96X128", 8, 384, 256, 7092),
    ("GEMM_SLOT_96X128", 8, 960, 768, 1000),
    ("GEMM_SLOT_64X128", 8, 700, 530, 600), ("GEMM_SLOT_64X128", 8, 65, 127, 256), ("GEMM_SLOT_64X128", 8, 384, 256, 7092),
]


@pytest.mark.parametrize("name,bits,M,N,K", VARIANT_CASES)
def test_gemm_every_variant_exact(gpu, name, bits, M, N, K):
    """Every GEMM kernel by name (hot_gemm_i8_variant): int32 accumulators bit-exact, and the
    dequantised output (the other store path: no int32 side output) equal to the epilogue formula."""
    from hot_amd import _lib, ops
    variant = getattr(_lib, name)
    a, b = rand_codes(M, K, bits, 31), rand_codes(N, K, bits, 32)
    kp = ops.kpad(K)
    rng = np.random.default_rng(33)
    sa = rng.uniform(1e-4, 2e-4, size=M).astype(np.float32)
    sb = rng.uniform(1e-3, 2e-3, size=1).astype(np.float32)
    A, B = to_operand(a, bits, kp).to(gpu), to_operand(b, bits, kp).to(gpu)
    acc_ref = exact_acc(a, b)
    assert np.array_equal(acc_ref, orc.int_gemm_nt(a, b))
    out, acc = ops.gemm_i8(A, B, K, bits, torch.from_numpy(sa).to(gpu), torch.from_numpy(sb).to(gpu), post_scale=1 / 16,
                           return_acc=True, variant=variant)
    ref = dequant_ref(acc_ref, sa, sb[0], 1 / 16)
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    assert np.array_equal(out.cpu().numpy(), ref)
    for dt in (torch.float32, torch.bfloat16):
        out2 = ops.gemm_i8(A, B, K, bits, torch.from_numpy(sa).to(gpu), torch.from_numpy(sb).to(gpu), post_scale=1 / 16,
                           out_dtype=dt, variant=variant)
        assert torch.equal(out2.cpu(), torch.from_numpy(ref).to(dt))


@pytest.mark.parametrize("bits,M,N,K,expect", [
    (8, 4000, 4090, 2048, "GEMM_SLOT_256"),        # 16 x 16 large tiles, ragged on both edges
    (4, 4000, 4090, 8192, "GEMM_SLOT_256"),
    (4, 4000, 4090, 8320, "GEMM_DMA_256_S4"),      # rows of 4160 bytes: not whole 128-byte lines
    (4, 5000, 6600, 192, "GEMM_DMA_128_S3"),       # short K: many small tiles, three workgroups per CU
    (8, 5000, 6600, 192, "GEMM_DMA_128_S4"),
    (8, 384, 256, 4000, "GEMM_SLOT_32X128"),       # few tiles: the shortest tile, 24 workgroups instead of 6
    (8, 3000, 800, 4000, "GEMM_SLOT_96X128"),      # 168 tiles of 128 x 128, 224 of 96 x 128, 329 of 64 x 128
    (8, 4096, 1024, 1024, "GEMM_SLOT_128"),        # 256 tiles: nothing shorter keeps one round
    (4, 384, 256, 4200, "GEMM_DMA_128_S4"),        # the same with rows of 2112 bytes
    (4, 12608, 768, 3072, "GEMM_SLOT_160X256"),    # ViT-B fc1 g_x: one balanced round of 237 tiles
])
def test_gemm_plan_and_result(gpu, bits, M, N, K, expect):
    """hot_gemm_i8 picks its kernel by the rule hot_gemm_plan reports; the test names the kernel it
    means to cover, so a change of the rule cannot silently move it to another one."""
    from hot_amd import _lib, ops
    assert ops.gemm_plan(M, N, K, bits) == getattr(_lib, expect)
    a, b = rand_codes(M, K, bits, 21), rand_codes(N, K, bits, 22)
    kp = ops.kpad(K)
    one = torch.ones(1, device=gpu)
    A, B = to_operand(a, bits, kp).to(gpu), to_operand(b, bits, kp).to(gpu)
    acc_ref = exact_acc(a, b)
    _, acc = ops.gemm_i8(A, B, K, bits, one, one, return_acc=True)
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    sa = torch.full((M,), 2.0 ** -9, device=gpu)
    out = ops.gemm_i8(A, B, K, bits, sa, one, post_scale=1 / 16, out_dtype=torch.bfloat16)    # the staged epilogue
    ref = torch.from_numpy(dequant_ref(acc_ref, np.full(M, 2.0 ** -9, np.float32), 1.0, 1 / 16)).to(torch.bfloat16)
    assert torch.equal(out.cpu(), ref)


@pytest.mark.parametrize("bits,M,N,K,expect", [
    (4, 8192, 4096, 11008, "GEMM_SLOT_256"),     # Llama-7B gate/up: g_x
    (8, 11008, 4096, 4096, "GEMM_SLOT_256"),     # Llama-7B gate/up: g_W at the paper rule (L' = 4096)
    (4, 8192, 11008, 4096, "GEMM_SLOT_256"),     # Llama-7B down: g_x
    (8, 4096, 11008, 4096, "GEMM_SLOT_256"),     # Llama-7B down: g_W
    (8, 4096, 4096, 4096, "GEMM_SLOT_256"),      # Llama-7B q/k/v/o: g_W
    (4, 8192, 4096, 4096, "GEMM_SLOT_256"),      # Llama-7B q/k/v/o: g_x
])
def test_gemm_llama_products_sampled_rows_and_columns(gpu, bits, M, N, K, expect):
    """The products of the Llama-7B shapes, on the kernel the library picks for them (named, so the
    test cannot drift off it), checked on whole sampled rows and whole sampled columns of the
    output, so that every output tile is touched: int32 accumulators and the bf16 results bit for bit."""
    from hot_amd import _lib, ops
    assert ops.gemm_plan(M, N, K, bits) == getattr(_lib, expect)
    a, b = rand_codes(M, K, bits, 41), rand_codes(N, K, bits, 42)
    kp = ops.kpad(K)
    A, B = to_operand(a, bits, kp).to(gpu), to_operand(b, bits, kp).to(gpu)
    rng = np.random.default_rng(43)
    sa = rng.uniform(1e-4, 2e-4, size=M).astype(np.float32)
    sb = np.float32(1.5e-3)
    rows = np.unique(np.concatenate([[0, 255, 256, M - 1], rng.integers(0, M, 40)]))
    cols = np.unique(np.concatenate([[0, 255, 256, N - 1], rng.integers(0, N, 40)]))
    acc_rows, acc_cols = exact_acc(a[rows], b), exact_acc(a, b[cols])
    out, acc = ops.gemm_i8(A, B, K, bits, torch.from_numpy(sa).to(gpu), torch.tensor([sb], device=gpu), post_scale=1 / 16,
                           return_acc=True)
    acc = acc.cpu().numpy()
    assert np.array_equal(acc[rows], acc_rows) and np.array_equal(acc[:, cols], acc_cols)
    del acc
    out16 = ops.gemm_i8(A, B, K, bits, torch.from_numpy(sa).to(gpu), torch.tensor([sb], device=gpu), post_scale=1 / 16,
                        out_dtype=torch.bfloat16).cpu()
    assert torch.equal(out16[rows], torch.from_numpy(dequant_ref(acc_rows, sa[rows], sb, 1 / 16)).to(torch.bfloat16))
    assert torch.equal(out16[:, cols], torch.from_numpy(dequant_ref(acc_cols, sa, sb, 1 / 16)).to(torch.bfloat16))
    assert np.array_equal(out.cpu().numpy()[rows], dequant_ref(acc_rows, sa[rows], sb, 1 / 16))


@pytest.mark.parametrize("M,N,K,bias,out_dtype", [
    (200, 96, 128, True, torch.float32),        # ragged tiles, direct epilogue
    (1000, 300, 384, False, torch.float32),     # 300 columns: four-wide stores across a ragged edge
    (512, 512, 1024, True, torch.bfloat16),     # whole tiles: the LDS-staged epilogue
    (12608, 768, 768, True, torch.bfloat16),    # ViT-B proj forward, the 160 x 256 tile
])
@pytest.mark.parametrize("variant", ["auto", "GEMM_SLOT_128", "GEMM_SLOT_256", "GEMM_SLOT_160X256"])
def test_gemm_bf16_forward_product(gpu, M, N, K, bias, out_dtype, variant):
    """hot_gemm_bf16 = x W^T + b (F.linear, utils/quant_matmul.py:173-176): bf16 operands are exact in
    float64, so the float64 product is the reference; an fp32 sum over K terms in any order lies within
    K 2^-24 sum|x w| of it (one rounding more for a bf16 output: 2^-8 relative)."""
    from hot_amd import _lib, ops
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    b = torch.randn(N, generator=g).to(out_dtype) if bias else None
    v = 0 if variant == "auto" else getattr(_lib, variant)
    y = ops.gemm_bf16(x.to(gpu), w.to(gpu), b.to(gpu) if bias else None, out_dtype=out_dtype, variant=v).cpu().double()
    ref = x.double() @ w.double().T
    mag = x.double().abs() @ w.double().abs().T
    if bias:
        ref = ref + b.double()
        mag = mag + b.double().abs()
    bound = K * 2.0 ** -24 * mag + (2.0 ** -8 * ref.abs() if out_dtype == torch.bfloat16 else 2.0 ** -23 * ref.abs())
    assert torch.all((y - ref).abs() <= bound)


def test_gemm_bf16_refuses_what_it_does_not_take(gpu):
    from hot_amd import ops
    x = torch.zeros(64, 100, device=gpu, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ops.gemm_bf16(x, x)
    with pytest.raises(RuntimeError, match="bf16 operands"):
        ops.gemm_bf16(x.float(), x.float())


def test_gemm_splits_rule():
    """hot_gemm_splits: products with few output tiles and a long K are cut, others are not."""
    from hot_amd import _lib
    f = _lib.lib().hot_gemm_splits
    assert f(3072, 768, 7092, 8) == 1          # ViT-B fc1 g_W: 192 tiles of 96 x 128, one deep-ring workgroup each
    assert f(768, 768, 7092, 8) == 1           # ViT-B proj g_W: 144 tiles of 32 x 128 instead of 36 tiles in 7 K ranges
    assert f(768, 768, 7092, 4) == 3           # the INT4 form of that product: 36 tiles, K cut into 3 ranges
    assert f(12608, 768, 3072, 4) == 1         # ViT-B fc1 g_x: 594 tiles
    assert f(11008, 4096, 4096, 8) == 1
    assert f(256, 256, 128, 8) == 1            # short K
    assert f(256, 256, 2304, 8) == 1           # INT8, 4 tiles of 128 x 128: 16 tiles of 32 x 128, unsplit
    assert _lib.lib().hot_gemm_workspace_bytes(256, 256, 2304, 8) == 4 * 2 * 128 * 128 * 4



@pytest.mark.parametrize("n,L,C,scale,rounding,dtype", [
    (128, 256, 72, "tensor", "nearest", torch.float32),
    (128, 512, 264, "row", "stoch", torch.bfloat16),
    (256, 512, 64, "sawb", "nearest", torch.float32),
    (1024, 2048, 40, "tensor", "stoch", torch.float32),
    (8192, 8192, 16, "tensor", "nearest", torch.bfloat16),
])
def test_hla_tokenwise_large_blocks(gpu, n, L, C, scale, rounding, dtype):
    """Blocks above 64 tokens (the make_WHT rule on token counts with many factors of two): 128 in
    registers, larger ones through the two-level path; codes, steps and the transposed layout must
    equal the one-pass oracle."""
    from hot_amd import ops
    nn_, rows = orc.hla_rows(n)
    assert nn_ == n
    x = (torch.randn(L, C, generator=torch.Generator().manual_seed(n + C)) * 0.5).to(dtype)
    mode = {"tensor": orc.SCALE_TENSOR, "row": orc.SCALE_ROW, "sawb": orc.SCALE_SAWB}[scale]
    rnd = orc.ROUND_STOCH if rounding == "stoch" else orc.ROUND_NEAREST
    tt = np.ascontiguousarray(orc.fwht_blocks_first(x.float().numpy(), n, rows).T)      # [C, L']
    q_ref, s_ref = orc.quant(tt, 8, mode, rnd, seed=3, stream=orc.STREAM_GW,
                             index=orc.colwise_rng_index(C, L // n, rows))
    codes, s, kout = ops.hla_tokenwise(x.to(gpu), n, list(rows), bits=8, rounding=rounding, scale=scale, seed=3)
    got = codes.cpu().numpy()
    assert kout == tt.shape[1]
    assert np.array_equal(s.cpu().numpy(), np.atleast_1d(s_ref).astype(np.float32).reshape(-1))
    assert np.array_equal(got[:, :kout], q_ref) and not got[:, kout:].any()


@pytest.mark.parametrize("n,L,C,scale,rounding,dtype", [
    (256, 768, 200, "tensor", "nearest", torch.float32),          # three blocks, ragged channel strip, run lengths not multiples of 4
    (256, 512, 64, "sawb", "stoch", torch.bfloat16),
    (1024, 2048, 136, "row", "stoch", torch.float32),
    (2048, 2048, 72, "tensor", "nearest", torch.float16),
    (8192, 8192, 80, "tensor", "stoch", torch.bfloat16),
])
def test_hla_tokenwise_large_blocks_run_major(gpu, n, L, C, scale, rounding, dtype):
    """The kept rows listed run by run (sorted by (row % 64, row // 64): hadamard_matmul.run_major, what the
    layers pass for blocks above 128 tokens): the quantise pass of the two-level path then stores K-major
    itself.  Codes in the caller's order, steps, zero padding and the numbering of stochastic rounding
    (by natural row, whatever the order of the list) equal the one-pass oracle; the same rows in the
    reference's sequency order give the same codes, permuted."""
    from hot_amd import ops
    from hot_amd.hadamard_matmul import run_major
    _, rows_seq = orc.hla_rows(n)
    rows = run_major(rows_seq)
    assert sorted(rows.tolist()) == sorted(rows_seq.tolist()) and not np.array_equal(rows, rows_seq)
    x = (torch.randn(L, C, generator=torch.Generator().manual_seed(n + C)) * 0.5).to(dtype)
    mode = {"tensor": orc.SCALE_TENSOR, "row": orc.SCALE_ROW, "sawb": orc.SCALE_SAWB}[scale]
    rnd = orc.ROUND_STOCH if rounding == "stoch" else orc.ROUND_NEAREST
    tt = np.ascontiguousarray(orc.fwht_blocks_first(x.float().numpy(), n, rows).T)      # [C, L']
    q_ref, s_ref = orc.quant(tt, 8, mode, rnd, seed=3, stream=orc.STREAM_GW,
                             index=orc.colwise_rng_index(C, L // n, rows))
    codes, s, kout = ops.hla_tokenwise(x.to(gpu), n, list(rows), bits=8, rounding=rounding, scale=scale, seed=3)
    got = codes.cpu().numpy()
    assert kout == tt.shape[1]
    assert np.array_equal(s.cpu().numpy(), np.atleast_1d(s_ref).astype(np.float32).reshape(-1))
    assert np.array_equal(got[:, :kout], q_ref) and not got[:, kout:].any()
    # the sequency order: the general path (codes through the workspace and a transpose), same codes permuted
    codes2, s2, _ = ops.hla_tokenwise(x.to(gpu), n, list(rows_seq), bits=8, rounding=rounding, scale=scale, seed=3)
    pos = {int(v): i for i, v in enumerate(rows)}
    perm = np.array([pos[int(v)] for v in rows_seq])
    r = len(rows)
    got2 = codes2.cpu().numpy()[:, :kout].reshape(C, L // n, r)
    assert np.array_equal(got2, got[:, :kout].reshape(C, L // n, r)[:, :, perm]) and torch.equal(s, s2)


@pytest.mark.parametrize("bits,rounding,dtype", [(8, "stoch", torch.bfloat16), (4, "nearest", torch.float32)])
def test_hla_tokenwise_block128_any_selection(gpu, bits, rounding, dtype):
    """A 128-token block with a selection that is not the make_WHT one (table read at run time),
    8-bit and 4-bit codes."""
    from hot_amd import ops
    n, L, C = 128, 384, 136
    rows = np.random.default_rng(5).permutation(n)[:50]
    x = (torch.randn(L, C, generator=torch.Generator().manual_seed(9)) * 0.5).to(dtype)
    rnd = orc.ROUND_STOCH if rounding == "stoch" else orc.ROUND_NEAREST
    tt = np.ascontiguousarray(orc.fwht_blocks_first(x.float().numpy(), n, rows).T)
    q_ref, s_ref = orc.quant(tt, bits, orc.SCALE_TENSOR, rnd, seed=3, stream=orc.STREAM_GW,
                             index=orc.colwise_rng_index(C, L // n, rows))
    codes, s, kout = ops.hla_tokenwise(x.to(gpu), n, [int(v) for v in rows], bits=bits, rounding=rounding,
                                       scale="tensor", seed=3)
    got = codes.cpu().numpy()
    assert s.cpu().numpy()[0] == np.float32(s_ref)
    assert np.array_equal(got[:, :kout], q_ref) and not got[:, kout:].any()
