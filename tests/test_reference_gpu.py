"""Each kernel against its plain C++ reference (csrc/host/reference.cpp), which takes its sums in the
order that the kernel's contract names: where the hardware's arithmetic is exact in that order (32-bit
projections), the bits must agree; elsewhere a hardware exponential or reciprocal square root stands
between them, and the tolerance is a few units of its last place, far below what another order of
summation would show."""
import numpy as np
import pytest
import torch

from vosti_amd.kernels import reference as ref

pytestmark = pytest.mark.gpu
F32, BF16 = torch.float32, torch.bfloat16
DTYPES = [F32, BF16]


def kern(dtype):
    from vosti_amd.kernels import kernels_for
    return kernels_for(dtype)


def rnd(*shape, seed=0, scale=1.0, dtype=F32):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def tol(dtype, f32=dict(rtol=2e-6, atol=2e-7)):
    return dict(rtol=2 ** -7, atol=2 ** -8) if dtype == BF16 else f32


def check(got, want, dtype, **kw):
    torch.testing.assert_close(got.float().cpu(), torch.from_numpy(np.asarray(want)), **tol(dtype, **kw))


@pytest.mark.parametrize("M,N,K", [(1, 40, 512), (5, 33, 520), (20, 100, 1040), (64, 72, 4608), (100, 130, 1536), (300, 140, 2056),
                                   (8, 6200, 1024)])
def test_projection_in_32_bit_is_the_reference_bit_for_bit(M, N, K):
    """Chunks of 512, slabs of 16, the four feeds of a slab, the products of a feed one after the other,
    each fused into the sum, the chunk sums added in order: whichever kernel takes the shape."""
    k = kern(F32)
    a, w = rnd(M, K, seed=1), rnd(N, K, seed=2, scale=0.1)
    want = ref.gemm(a.numpy(), w.numpy(), bf16=False)
    for kernel in (0, 2, 3):
        got = k.gemm(a.cuda(), w.cuda(), kernel=kernel).cpu().numpy()
        assert np.array_equal(got, want), (kernel, np.abs(got - want).max())


@pytest.mark.parametrize("M,N,K", [(3, 40, 512), (20, 100, 1040), (130, 72, 4608)])
def test_projection_in_bfloat16(M, N, K):
    k = kern(BF16)
    a, w = rnd(M, K, seed=1, dtype=BF16), rnd(N, K, seed=2, scale=0.1, dtype=BF16)
    check(k.gemm(a.cuda(), w.cuda()), ref.gemm(a.float().numpy(), w.float().numpy(), bf16=True), BF16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norms_swiglu_embedding(dtype):
    k, bf = kern(dtype), dtype == BF16
    x, r = rnd(7, 520, seed=3, dtype=dtype), rnd(7, 520, seed=4, dtype=dtype)
    w = (1 + 0.1 * rnd(520, seed=5)).to(dtype)
    check(k.rmsnorm(x.cuda(), w.cuda(), 1e-5), ref.rmsnorm(x.float().numpy(), w.float().numpy(), 1e-5, bf), dtype)
    res = r.clone().cuda()
    got = k.add_rmsnorm(x.cuda(), res, w.cuda(), 1e-6)
    n, new_res = ref.add_rmsnorm(x.float().numpy(), r.float().numpy(), w.float().numpy(), 1e-6, bf)
    check(got, n, dtype)
    assert np.array_equal(res.float().cpu().numpy(), new_res)
    gu = rnd(9, 2 * 130, seed=6, scale=2.0, dtype=dtype)
    check(k.swiglu(gu.cuda()), ref.swiglu(gu.float().numpy(), bf), dtype, f32=dict(rtol=1e-5, atol=1e-6))
    table, ids = rnd(50, 24, seed=7, dtype=dtype), torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    assert np.array_equal(k.embedding(table.cuda(), ids.cuda()).float().cpu().numpy(), ref.embedding(table.float().numpy(), ids.numpy()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,rot", [(4, 2, 16, 8), (8, 2, 128, 128), (3, 1, 80, 80)])
def test_head_norm_rotation_and_store(dtype, nq, nkv, d, rot):
    k, bf = kern(dtype), dtype == BF16
    T, P, pages = 9, 8, 5
    qkv = rnd(T, (nq + 2 * nkv) * d, seed=8, dtype=dtype)
    qw, kw = (1 + 0.1 * rnd(d, seed=9)).to(dtype), (1 + 0.1 * rnd(d, seed=10)).to(dtype)
    inv = 1.0 / (1e4 ** (torch.arange(0, rot, 2, dtype=torch.int64).float() / rot))
    cos, sin = k.rope_tables(inv.cuda(), 64)
    pos = torch.tensor([0, 1, 5, 17, 40, 41, 63, 2, 3], dtype=torch.int32)
    slots = torch.tensor([5, -1, 12, 0, 23, 39, 8, -1, 31], dtype=torch.int32)
    kc, vc = torch.full((pages, nkv, P, d), 7.0, dtype=dtype), torch.full((pages, nkv, d, P), 7.0, dtype=dtype)
    kc_g, vc_g = kc.cuda(), vc.cuda()
    q = k.qkv_post(qkv.cuda(), nq=nq, nkv=nkv, d=d, q_out=None, k_cache=kc_g, v_cache=vc_g, page_size=P, q_w=qw.cuda(),
                   k_w=kw.cuda(), eps=1e-5, cos=cos, sin=sin, positions=pos.cuda(), slots=slots.cuda())
    kc_r, vc_r = kc.float().numpy().copy(), vc.float().numpy().copy()
    q_r = ref.qkv_post(qkv.float().numpy(), nq=nq, nkv=nkv, d=d, k_cache=kc_r, v_cache=vc_r, page_size=P,
                       q_w=qw.float().numpy(), k_w=kw.float().numpy(), eps=1e-5, cos=cos.float().cpu().numpy(),
                       sin=sin.float().cpu().numpy(), positions=pos.numpy(), slots=slots.numpy(), bf16=bf)
    check(q, q_r, dtype, f32=dict(rtol=1e-5, atol=1e-6))
    check(kc_g, kc_r, dtype, f32=dict(rtol=1e-5, atol=1e-6))
    assert np.array_equal(vc_g.float().cpu().numpy(), vc_r)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,P,window", [(4, 2, 16, 16, 0), (8, 2, 128, 64, 0), (6, 1, 64, 64, 300), (2, 2, 80, 32, 0)])
def test_attention_folds_in_the_reference_order(dtype, nq, nkv, d, P, window):
    """Prompt rows and decoded rows, lengths over several tiles and segments.  In 32-bit the kernels and
    the reference differ by the hardware's 2^x only: a few parts in ten million, where a fold in another
    order (tiles straight into the total, a running maximum) shows at a part in a million and more."""
    from test_kernels_gpu import build_cache, run_attention
    k, bf = kern(dtype), dtype == BF16
    shapes = [(70, 70), (1, 600), (33, 1100), (1, 257), (130, 385)]
    q_list = [rnd(ql, nq, d, seed=10 + i, dtype=dtype) for i, (ql, kl) in enumerate(shapes)]
    kk = [rnd(kl, nkv, d, seed=30 + i, dtype=dtype) for i, (ql, kl) in enumerate(shapes)]
    vv = [rnd(kl, nkv, d, seed=50 + i, dtype=dtype) for i, (ql, kl) in enumerate(shapes)]
    got = run_attention(k, q_list, kk, vv, P, dtype, window=window, seed=3)
    n_pages = sum(-(-x.shape[0] // P) for x in kk) + 3
    kc, vc, table = build_cache(kk, vv, P, n_pages, 3, dtype, None)
    cu = np.cumsum([0] + [ql for ql, _ in shapes])
    want = ref.paged_attention(torch.cat(q_list).float().numpy(), kc.float().numpy(), vc.float().numpy(), table.numpy(), cu,
                               [kl for _, kl in shapes], scale=d ** -0.5, window=window, bf16=bf)
    check(got, want, dtype, f32=dict(rtol=2e-6, atol=5e-7))


@pytest.mark.parametrize("dtype", DTYPES)
def test_sampler(dtype):
    k = kern(dtype)
    V = 5003
    logits = rnd(6, V, seed=60, scale=2.5, dtype=dtype)
    assert k.sample(logits.cuda()).cpu().tolist() == [ref.argmax(r) for r in logits.float().numpy()]
    temps = torch.tensor([0.7, 1.3, 0.0, 0.2, 2.0, 0.9])
    unis = torch.tensor([0.013, 0.5, 0.4, 0.77, 0.999, 0.31])
    got = k.sample(logits.cuda(), temps.cuda(), unis.cuda()).cpu().tolist()
    want = [ref.sample(r, float(t), float(u)) for r, t, u in zip(logits.float().numpy(), temps, unis)]
    assert got == want
