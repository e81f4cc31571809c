"""The plain C++ references of the kernels (csrc/host/reference.cpp) against the plain Python
implementation: two independent writings of the same formulas."""
import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from vosti_amd.kernels import reference as ref

F32, BF16 = torch.float32, torch.bfloat16


def rnd(*shape, seed=0, scale=1.0, dtype=F32):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype).float()


def close(a, b, bf16):
    # The two differ by the order of their sums: a step of the type where a value lands on a neighbour.
    tol = dict(rtol=2 ** -7, atol=2 ** -8) if bf16 else dict(rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(torch.as_tensor(np.asarray(a)), torch.as_tensor(np.asarray(b)), **tol)


def test_rounding_to_bfloat16_is_nearest_even():
    for x in (1.0, 1.00390625, 1.01171875, -3.1415927, 1e-30, 65504.0, 0.1, -0.0, 3.3895314e38):
        assert ref.round_bf16(x) == torch.tensor(x, dtype=F32).bfloat16().float().item(), x
    assert np.isinf(ref.round_bf16(float("inf"))) and np.isnan(ref.round_bf16(float("nan")))


@pytest.mark.parametrize("bf16", [False, True])
def test_elementwise_references(bf16):
    dt = BF16 if bf16 else F32
    table, ids = rnd(11, 6, dtype=dt), torch.tensor([3, 0, 10, 3], dtype=torch.int32)
    assert np.array_equal(ref.embedding(table.numpy(), ids.numpy()), plain.embedding(ids, table).numpy())
    x, r, w = rnd(5, 72, seed=1, dtype=dt), rnd(5, 72, seed=2, dtype=dt), (1 + 0.1 * rnd(72, seed=3)).to(dt).float()
    close(ref.rmsnorm(x.numpy(), w.numpy(), 1e-5, bf16), plain.rms_norm(x, w, 1e-5, dt), bf16)
    n, res = ref.add_rmsnorm(x.numpy(), r.numpy(), w.numpy(), 1e-6, bf16)
    pn, pr = plain.add_rms_norm(x, r, w, 1e-6, dt)
    close(n, pn, bf16)
    assert np.array_equal(res, pr.numpy())                   # one addition, one rounding: no order to differ in
    gu = rnd(4, 20, seed=4, scale=2.0, dtype=dt)
    close(ref.swiglu(gu.numpy(), bf16), plain.swiglu(gu, dt), bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("M,N,K", [(3, 5, 64), (2, 7, 520), (4, 3, 1040)])
def test_gemm_reference(bf16, M, N, K):
    dt = BF16 if bf16 else F32
    a, w = rnd(M, K, seed=5, dtype=dt), rnd(N, K, seed=6, scale=0.1, dtype=dt)
    close(ref.gemm(a.numpy(), w.numpy(), bf16), plain.linear(a, w, dt), bf16)
    # The order is a function of K only: a row alone gives the bits it has in the batch.
    assert np.array_equal(ref.gemm(a.numpy()[1:2], w.numpy(), bf16)[0], ref.gemm(a.numpy(), w.numpy(), bf16)[1])


@pytest.mark.parametrize("bf16", [False, True])
def test_qkv_post_reference(bf16):
    dt = BF16 if bf16 else F32
    T, nq, nkv, d, P, pages = 5, 4, 2, 16, 4, 6
    qkv = rnd(T, (nq + 2 * nkv) * d, seed=7, dtype=dt)
    qw, kw = (1 + 0.1 * rnd(d, seed=8)).to(dt).float(), (1 + 0.1 * rnd(d, seed=9)).to(dt).float()
    cos, sin = plain.rope_tables(64, 8, 1e4, dt)              # a partial rotation: the first 8 of 16
    pos = torch.tensor([0, 3, 17, 40, 41], dtype=torch.int32)
    slots = torch.tensor([5, -1, 12, 0, 23], dtype=torch.int32)
    kc, vc = np.full((pages, nkv, P, d), 7.0, dtype=np.float32), np.full((pages, nkv, d, P), 7.0, dtype=np.float32)
    q = ref.qkv_post(qkv.numpy(), nq=nq, nkv=nkv, d=d, k_cache=kc, v_cache=vc, page_size=P, q_w=qw.numpy(), k_w=kw.numpy(),
                     eps=1e-5, cos=cos.numpy(), sin=sin.numpy(), positions=pos.numpy(), slots=slots.numpy(), bf16=bf16)
    x = qkv.view(T, nq + 2 * nkv, d)
    pq = plain.apply_rope(plain.head_rms_norm(x[:, :nq], qw, 1e-5, dt), cos, sin, pos, dt)
    pk = plain.apply_rope(plain.head_rms_norm(x[:, nq:nq + nkv], kw, 1e-5, dt), cos, sin, pos, dt)
    close(q, pq, bf16)
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        close(kc[s // P, :, s % P, :], pk[t], bf16)
        assert np.array_equal(vc[s // P, :, :, s % P], x[t, nq + nkv:].numpy())      # values are stored as they come
    untouched = np.ones((pages, P), dtype=bool)
    for s in slots.tolist():
        if s >= 0:
            untouched[s // P, s % P] = False
    assert (kc.transpose(0, 2, 1, 3)[untouched] == 7.0).all() and (vc.transpose(0, 3, 1, 2)[untouched] == 7.0).all()


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("window", [0, 70])
def test_attention_reference(bf16, window):
    """Prompt rows and a decoded row over pages in a shuffled order, lengths past a tile and a segment."""
    dt = BF16 if bf16 else F32
    nq, nkv, d, P = 4, 2, 16, 16
    shapes = [(5, 5), (1, 300), (40, 270), (3, 64)]
    n_pages = sum(-(-k // P) for _, k in shapes) + 1
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(1)).tolist()
    kc, vc = np.full((n_pages, nkv, P, d), np.nan, dtype=np.float32), np.full((n_pages, nkv, d, P), np.nan, dtype=np.float32)
    width = max(-(-k // P) for _, k in shapes)
    table = np.full((len(shapes), width), order[-1], dtype=np.int32)
    qs, refs, cu, klen = [], [], [0], []
    for s, (ql, kl) in enumerate(shapes):
        q, k, v = rnd(ql, nq, d, seed=10 + s, dtype=dt), rnd(kl, nkv, d, seed=20 + s, dtype=dt), rnd(kl, nkv, d, seed=30 + s, dtype=dt)
        for j in range(-(-kl // P)):
            page = order.pop(0)
            table[s, j] = page
            n = min(P, kl - j * P)
            kc[page, :, :n] = k[j * P:j * P + n].permute(1, 0, 2).numpy()
            vc[page, :, :, :n] = v[j * P:j * P + n].permute(1, 2, 0).numpy()
        qs.append(q)
        refs.append(plain.attention(q, k, v, d ** -0.5, dt, window=window))
        cu.append(cu[-1] + ql)
        klen.append(kl)
    got = ref.paged_attention(torch.cat(qs).numpy(), kc, vc, table, cu, klen, scale=d ** -0.5, window=window, bf16=bf16)
    close(got, torch.cat(refs), bf16)


def test_sampler_reference():
    # python/tests/test_qwen3_kernel_contracts.py:525-539: ties go to the first index, a NaN counts as the maximum.
    rows = np.array([[-3.0, 7.0, 7.0, 2.0], [np.nan, 5.0, np.nan, 1.0], [-np.inf, np.inf, 4.0, np.inf]], dtype=np.float32)
    assert [ref.argmax(r) for r in rows] == [1, 0, 1] and ref.argmax(np.empty(0, dtype=np.float32)) == 0
    assert ref.argmax(np.full(5, -np.inf, dtype=np.float32)) == 0
    row = rnd(3000, seed=40, scale=2.0).numpy()
    assert ref.sample(row, 0.0, 0.3) == ref.argmax(row) == int(np.argmax(row))
    p = torch.softmax(torch.from_numpy(row).double() / 0.7, 0)
    cdf = torch.cumsum(p, 0)
    for u in (0.0, 0.013, 0.5, 0.77, 0.999999):
        tok = ref.sample(row, 0.7, u)
        lo = cdf[tok - 1].item() if tok else 0.0
        assert lo - 1e-5 <= u <= cdf[tok].item() + 1e-5, (u, tok)
    assert ref.sample(row, 1e-4, 0.9) == ref.argmax(row)         # temperature -> 0 is greedy
