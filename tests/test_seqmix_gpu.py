"""Numerics of the sequence-mixer HIP kernels (csrc/kernels/seqmix.hip, latent.hip, the squared-ReLU
expert mode of moe.hip) against the plain-PyTorch f32 references of the same ops (ops.reference),
in bf16 and f32, over packed batches of unequal sequences that continue from state slots."""
import pytest
import torch

from distributed_llm_amd import ops
from distributed_llm_amd.ops import reference as ref
from distributed_llm_amd.ops import seqmix

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.bfloat16, torch.float32]


@pytest.fixture(autouse=True, scope="module")
def _native():
    assert ops.native_available(), "HIP extension must be built for GPU tests"


def tol(dt):
    return dict(atol=2e-2, rtol=2e-2) if dt == torch.bfloat16 else dict(atol=2e-5, rtol=2e-5)


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def batch(qlens, starts):
    """Packed metadata of sequences with ``qlens`` new tokens after ``starts`` old ones; slots are
    given out of order on purpose."""
    qstart, t = [], 0
    for n in qlens:
        qstart.append(t)
        t += n
    ctx = [a + n for a, n in zip(starts, qlens)]
    rows = list(reversed(range(len(qlens))))
    pos = [p for a, n in zip(starts, qlens) for p in range(a, a + n)]
    return t, i32(qstart), i32(qlens), i32(ctx), i32(rows), i32(pos)


CASES = [([5, 1, 0, 19], [0, 7, 3, 2]), ([1, 1, 1], [4, 0, 33]), ([70], [0]), ([2, 3], [1, 0])]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n", [24, 104, 328, 1000])
def test_rms_rows_and_resadd(dt, n):
    torch.manual_seed(0)
    x = torch.randn(13, n + 8, device=DEV).to(dt)[:, 3:3 + n]      # a column slice
    w = torch.randn(n, device=DEV)
    torch.testing.assert_close(seqmix.rms_rows(x, w, 1e-6).float(), ref.rms_rows(x, w, 1e-6).float(), **tol(dt))
    torch.testing.assert_close(seqmix.rms_rows(x, None, 1e-5, torch.float32), ref.rms_rows(x, None, 1e-5, torch.float32),
                               atol=1e-5, rtol=1e-5)
    y = torch.randn(13, n, device=DEV).to(dt)
    r1 = torch.randn(13, n, device=DEV)
    r2 = r1.clone()
    l1 = torch.empty(13, n, device=DEV, dtype=dt) if dt == torch.bfloat16 else None
    l2 = l1.clone() if l1 is not None else None
    seqmix.norm_resadd(y, w, 1e-6, r1, l1)
    ref.norm_resadd(y, w, 1e-6, r2, l2)
    torch.testing.assert_close(r1, r2, atol=1e-5, rtol=1e-5)
    if l1 is not None:
        torch.testing.assert_close(l1.float(), l2.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("C,N,K,R", [(40, 20, 3, 5), (128, 16, 4, 8), (72, 1, 2, 3), (64, 40, 1, 4)])
def test_conv_and_scan(dt, case, C, N, K, R):
    torch.manual_seed(1)
    qlens, starts = case
    T, qstart, qlen, ctx, rows, _ = batch(qlens, starts)
    slots = len(qlens) + 1
    xz = torch.randn(T, 2 * C, device=DEV).to(dt)
    w, b = torch.randn(C, K, device=DEV) * 0.5, torch.randn(C, device=DEV) * 0.1
    conv0 = torch.randn(slots, K - 1, C, device=DEV).to(dt)
    ssm0 = torch.randn(slots, C, N, device=DEV)
    y = seqmix.causal_conv_silu(xz, w, b, conv0, qstart, qlen, ctx, rows)
    yr = ref.causal_conv_silu(xz, w, b, conv0, qstart, qlen, ctx, rows)
    torch.testing.assert_close(y.float(), yr.float(), **tol(dt))
    dbc = torch.randn(T, R + 2 * N + 3, device=DEV).to(dt)[:, :R + 2 * N]
    dt_raw = (torch.randn(T, C, device=DEV) * 2).to(dt)
    dtb = torch.randn(C, device=DEV)
    A = -torch.exp(torch.randn(C, N, device=DEV))
    D = torch.randn(C, device=DEV)
    c1, s1, c2, s2 = conv0.clone(), ssm0.clone(), conv0.clone(), ssm0.clone()
    o1 = seqmix.selective_scan(yr, dt_raw, dtb, A, dbc, R, D, xz, s1, c1, qstart, qlen, ctx, rows)
    o2 = ref.selective_scan(yr, dt_raw, dtb, A, dbc, R, D, xz, s2, c2, qstart, qlen, ctx, rows)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dt))
    torch.testing.assert_close(s1, s2, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(c1.float(), c2.float(), atol=0, rtol=0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("H,d,dv,rot", [(2, 64, 48, 32), (3, 32, 24, 16), (1, 16, 80, 0), (4, 128, 128, 64)])
def test_retention(dt, case, H, d, dv, rot, chunked):
    torch.manual_seed(2)
    qlens, starts = case
    T, qstart, qlen, ctx, rows, pos = batch(qlens, starts)
    qkvg = torch.randn(T, 2 * H * d + 2 * H * dv, device=DEV).to(dt)
    table = ops.rope_cos_sin(128, max(rot, 2), 10000.0, DEV)
    decay = torch.tensor([1.0 - 2.0 ** (-2 - h) for h in range(H)], device=DEV)
    st0 = torch.randn(len(qlens) + 1, H, d, dv, device=DEV)
    s1, s2 = st0.clone(), st0.clone()
    o1 = seqmix.retention(qkvg, H, d, dv, table, rot, decay, s1, 1e-6, pos, qstart, qlen, ctx, rows, chunked=chunked)
    o2 = ref.retention(qkvg, H, d, dv, table, rot, decay, s2, 1e-6, pos, qstart, qlen, ctx, rows)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dt))
    torch.testing.assert_close(s1, s2, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("splits", [1, 3, 16])
@pytest.mark.parametrize("mfma", [False, True, 32])
@pytest.mark.parametrize("H,dim,rot,rank", [(8, 32, 16, 96), (3, 16, 8, 40), (20, 32, 16, 128), (1, 8, 64, 512), (2, 8, 6, 70)])
def test_latent_attention(dt, case, H, dim, rot, rank, splits, mfma):
    if mfma and dt != torch.bfloat16:
        pytest.skip("the matrix-core kernel serves bf16 models")
    wg_rows = 32 if mfma == 32 else 16
    torch.manual_seed(3)
    qlens, starts = case
    T, qstart, qlen, ctx, rows, pos = batch(qlens, starts)
    S, nblk = len(qlens), 12
    table = ops.rope_cos_sin(256, rot, 10000.0, DEV)
    perm = torch.randperm(S * nblk, device=DEV).to(torch.int32).view(S, nblk)       # scattered pages
    cache1 = torch.zeros(S * nblk, 16, rank + rot, device=DEV, dtype=dt)
    cache2 = cache1.clone()
    # every sequence's earlier tokens, then this step's, through the cache-write kernel
    for lo, hi in ((0, None), (None, 0)):
        ps, sl = [], []
        for s, (a, n) in enumerate(zip(starts, qlens)):
            rng = range(0, a) if hi is None else range(a, a + n)
            for p_ in rng:
                ps.append(p_)
                sl.append(int(perm[s, p_ // 16]) * 16 + p_ % 16)
        if not ps:
            continue
        ckv = torch.randn(len(ps), rank + rot + 5, device=DEV).to(dt)[:, 5:]
        wn = torch.rand(rank, device=DEV) + 0.5
        seqmix.latent_kv_write(ckv, rank, wn, 1e-6, i32(ps), table, i32(sl), cache1)
        ref.latent_kv_write(ckv, rank, wn, 1e-6, i32(ps), table, i32(sl), cache2)
    torch.testing.assert_close(cache1.float(), cache2.float(), **tol(dt))
    qa = (torch.randn(H, T, rank, device=DEV) * 0.3).to(dt)
    q = torch.randn(T, H * (dim + rot), device=DEV).to(dt)
    from distributed_llm_amd.models.llama import AttnMeta
    meta = AttnMeta(slots=None, block_tables=perm, qstart=qstart, qlen=qlen, ctx=ctx, tile_seq=None, tile_tok0=None,
                    last_idx=None, host_qlen=qlens)
    ts, tt = meta.latent_tiles(H, DEV, wg_rows)
    o1 = seqmix.latent_attention(qa, q, dim, rot, pos, table, cache2, perm, qstart, qlen, ctx, ts, tt, 0.2, splits=splits, mfma=bool(mfma), rows=wg_rows)
    o2 = ref.latent_attention(qa, q, dim, rot, pos, table, cache2, perm, qstart, qlen, ctx, 0.2)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
def test_relu2_and_dense_gate(dt):
    torch.manual_seed(4)
    T, E, ff, k = 9, 6, 20, 3
    x = torch.randn(T, E * ff, device=DEV).to(dt)
    ids = torch.stack([torch.randperm(E, device=DEV)[:k] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, k, device=DEV)
    g = seqmix.dense_gate(ids, w, E)
    torch.testing.assert_close(g, ref.dense_gate(ids, w, E))
    torch.testing.assert_close(seqmix.relu2_scale(x, g, ff).float(), ref.relu2_scale(x, g, ff).float(), **tol(dt))
    torch.testing.assert_close(seqmix.relu2_scale(x).float(), ref.relu2_scale(x).float(), **tol(dt))


@pytest.mark.parametrize("T", [1, 7, 200])
def test_moe_relu2_grouped(T):
    torch.manual_seed(5)
    H, I, E, k = 256, 96, 6, 2
    x = (torch.randn(T, H, device=DEV)).to(torch.bfloat16)
    w1 = (torch.randn(E, I, H, device=DEV) * H ** -0.5).to(torch.bfloat16)
    w2 = (torch.randn(E, H, I, device=DEV) * I ** -0.5).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, device=DEV)[:k] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, k, device=DEV)
    assert seqmix.moe_ffn_relu2_ok(x, w1)
    y = seqmix.moe_ffn_relu2(x, ids, w, w1, w2)
    torch.testing.assert_close(y.float(), ref.moe_ffn_relu2(x, ids, w, w1, w2).float(), atol=3e-2, rtol=3e-2)
