"""Each kernel alone against its plain reference, at sizes other than the engine's."""
import math

import pytest
import torch

import plain_qwen3 as plain
from vosti_amd.kernels.ops import ATTN_ITEM_ROWS

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def kern(dtype):
    from vosti_amd.kernels import kernels_for
    return kernels_for(dtype)


def tol(dtype):
    # bfloat16: the plain function rounds where the kernel does, so the two differ where a sum taken in
    # another order lands on the neighbouring value: one step of the type (2^-8 to 2^-7 of the value),
    # and as much of the operands' size where the value is a difference of them.
    return dict(rtol=2 ** -7, atol=2 ** -8) if dtype == torch.bfloat16 else dict(rtol=2e-5, atol=2e-5)


def rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 503, 96), (17, 224, 96), (64, 256, 224), (16, 48, 520),
                                   (65, 130, 520), (130, 96, 1032), (300, 520, 2056), (8, 40, 4104),
                                   (8, 4100, 1024), (3, 72, 512), (33, 200, 1536), (64, 4096, 4608), (17, 90, 5120),
                                   (40, 6200, 1024), (64, 6144, 512), (23, 24, 2048), (48, 24700, 512), (20, 24576, 1024), (31, 6200, 4096), (17, 100, 1536), (9, 130, 12288), (16, 72, 8704), (2, 40, 5120), (100, 200, 1024), (65, 4100, 512), (130, 96, 1536),
                                   (250, 8200, 512), (129, 300, 4608), (300, 8400, 128), (700, 9000, 64), (300, 520, 2048), (520, 1000, 4096),
                                   (7, 600, 2560), (16, 1000, 3072), (9, 4200, 6144), (3, 264, 5632), (8, 300, 7168), (12, 90, 3584)])
def test_gemm(dtype, M, N, K):
    k = kern(dtype)
    a, w = rand((M, K), dtype, 1), rand((N, K), dtype, 2, 0.1)
    ref = (a.double() @ w.double().t()).float()
    got_t = k.gemm(a.cuda(), w.cuda(), kernel=2)
    torch.testing.assert_close(got_t.float().cpu(), ref.to(dtype).float(), **tol(dtype))
    if K % (64 if dtype == torch.bfloat16 else 32) == 0:
        for code, rows in ((13, 64), (15, 96), (16, 160)):
            assert torch.equal(k.gemm(a.cuda(), w.cuda(), kernel=code), got_t), f"{rows} weight rows per workgroup"
    if 64 < M <= 512 and K % 512 == 0:
        for code in (0, 8, 9, 10, 12):  # blocks of 64 (12: of 32) rows through the kernels that share activations through LDS
            assert torch.equal(k.gemm(a.cuda(), w.cuda(), kernel=code), got_t), code
    if M <= 64:
        codes = [1, 7, 0]           # one and two weight tiles per workgroup, and the kernel chosen by size
        if M > 16 and K % 512 == 0:
            codes += [8, 9, 10, 12] # activations shared through LDS: two, four and one chunk in work; 12: blocks of 32 rows
        if 16 < M <= 32 and K % 512 == 0 and K <= 4096 and dtype == torch.bfloat16:
            codes += [11]           # two activation tiles resident in registers
        for code in codes:
            got_s = k.gemm(a.cuda(), w.cuda(), kernel=code)
            assert torch.equal(got_s, got_t), f"the skinny kernel {code} and the tiled kernel must agree bitwise"
        # The route through chunk sums in a workspace (up to 64 rows of 16-bit elements, K in whole chunks).
        need = k.gemm_workspace_floats(M, N, K, force=True)
        assert (need > 0) == (K % 512 == 0 and dtype == torch.bfloat16)
        if need:
            ws = torch.full((need + 5,), float("nan"), device="cuda")       # what a call before may have left
            assert torch.equal(k.gemm(a.cuda(), w.cuda(), kernel=14, workspace=ws), got_t), "chunk sums"
            with pytest.raises(Exception, match="workspace"):
                k.gemm(a.cuda(), w.cuda(), kernel=14, workspace=ws[:need - 1])
    # A row of a batch equals the same row alone, bitwise.
    for r in {0, M // 2, M - 1}:
        one = k.gemm(a[r:r + 1].cuda(), w.cuda())
        assert torch.equal(one[0], got_t[r])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(2048, 5120, 512), (1024, 6144, 512), (4096, 5120, 576), (2000, 5000, 512), (1000, 6100, 640),
                                   (2048, 10240, 256), (1536, 6144, 512)])
def test_tile_width_chosen_by_rounds(dtype, M, N, K):
    """Row and column counts at which the tile kernel is given 96 or 160 weight rows a workgroup instead of 128
    (the last round of workgroups would otherwise run nearly empty), whole and with partial blocks in both
    directions: the same bits as with 128, whichever width is named or chosen, and right."""
    k = kern(dtype)
    a, w = rand((M, K), dtype, 1), rand((N, K), dtype, 2, 0.1)
    ref = (a.double() @ w.double().t()).float()
    square = k.gemm(a.cuda(), w.cuda(), kernel=4)
    torch.testing.assert_close(square.float().cpu(), ref.to(dtype).float(), **tol(dtype))
    for code in (0, 2, 13, 15, 16):
        assert torch.equal(k.gemm(a.cuda(), w.cuda(), kernel=code), square), code


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,K", [(4096, 4096), (6144, 1536), (8200, 1024), (24600, 512), (5120, 5120), (300, 8704), (130, 200),
                                 (520, 2560), (264, 6144)])
def test_gemm_every_row_count(dtype, N, K):
    """The kernel is chosen by the sizes, with many borders along the row count (16, 32, 40, 64, 128,
    256, ...): the first M rows of a product are the same bits whatever M is, and so are the fused
    gate/up rows."""
    k = kern(dtype)
    a, w = rand((330, K), dtype, 5).cuda(), rand((N, K), dtype, 6, K ** -0.5).cuda()
    full = k.gemm(a, w, kernel=2)
    torch.testing.assert_close(full.float().cpu(), (a.double().cpu() @ w.double().cpu().t()).to(dtype).float(), **tol(dtype))
    fused = k.gemm_swiglu(a, w) if N % 2 == 0 else None
    ws = torch.empty(1 << 24, device="cuda")      # enough for the route through chunk sums at every size here
    for M in list(range(1, 70)) + [95, 96, 97, 127, 128, 129, 191, 192, 193, 255, 256, 257, 300, 330]:
        assert torch.equal(k.gemm(a[:M], w), full[:M]), M
        assert torch.equal(k.gemm(a[:M], w, workspace=ws), full[:M]), M       # the kernel chosen when there is a workspace
        if fused is not None:
            assert torch.equal(k.gemm_swiglu(a[:M], w), fused[:M]), M
            if k.gemm_workspace_floats(M, N, K, swiglu=True, force=True):
                assert torch.equal(k.gemm_swiglu(a[:M], w, workspace=ws, split=True), fused[:M]), M


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_fused_qkv_equals_three(dtype):
    # The reference holds this bitwise (kernels/tests/runtime/test_qkv_matmul.py:20-34).
    k = kern(dtype)
    a = rand((37, 96), dtype, 3).cuda()
    ws = [rand((n, 96), dtype, 4 + i, 0.1).cuda() for i, n in enumerate((256, 64, 64))]
    fused = k.gemm(a, torch.cat(ws).contiguous())
    three = torch.cat([k.gemm(a, w) for w in ws], dim=1)
    assert torch.equal(fused, three)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_refuses_bad_width(dtype):
    from vosti_amd.kernels.ops import KernelError
    k = kern(dtype)
    with pytest.raises(KernelError, match="multiple"):
        k.gemm(rand((2, 50), dtype, 0).cuda(), rand((8, 50), dtype, 1).cuda())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H", [(1, 64), (7, 96), (33, 100), (5, 4104), (3, 17), (4, 2048), (2, 12288), (9, 4096)])
def test_rmsnorm_and_add(dtype, T, H):
    k = kern(dtype)
    x, r, w = rand((T, H), dtype, 1), rand((T, H), dtype, 2), (1 + 0.1 * rand((H,), torch.float32, 3)).to(dtype)
    eps = 1e-5
    got = k.rmsnorm(x.cuda(), w.cuda(), eps)
    torch.testing.assert_close(got.float().cpu(), plain.rms_norm(x, w, eps, dtype), **tol(dtype))
    res = r.clone().cuda()
    got = k.add_rmsnorm(x.cuda(), res, w.cuda(), eps)
    ref_n, ref_r = plain.add_rms_norm(x, r, w, eps, dtype)
    torch.testing.assert_close(got.float().cpu(), ref_n, **tol(dtype))
    torch.testing.assert_close(res.float().cpu(), ref_r, **tol(dtype))
    # Norm weights stored in 32-bit stay so.
    got32 = k.rmsnorm(x.cuda(), w.float().cuda(), eps)
    torch.testing.assert_close(got32.float().cpu(), plain.rms_norm(x, w, eps, dtype), **tol(dtype))
    # Row of a batch == the row alone.
    assert torch.equal(k.rmsnorm(x[T // 2: T // 2 + 1].cuda(), w.cuda(), eps)[0], k.rmsnorm(x.cuda(), w.cuda(), eps)[T // 2])


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_unit_rms(dtype):
    # With w = 1 and eps = 0 every row has unit RMS, whatever its scale.
    k = kern(dtype)
    x = (rand((4, 256), torch.float32, 5) * torch.tensor([[1e-2], [1.0], [30.0], [1e3]])).to(dtype)
    y = k.rmsnorm(x.cuda(), torch.ones(256, dtype=dtype).cuda(), 0.0).float()
    torch.testing.assert_close((y * y).mean(dim=1).sqrt().cpu(), torch.ones(4), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(3, 128), (9, 224), (2, 101)])
def test_swiglu(dtype, T, I):
    k = kern(dtype)
    gu = rand((T, 2 * I), dtype, 1, 2.0)
    ref = torch.nn.functional.silu(gu[:, :I].float()) * gu[:, I:].float()
    torch.testing.assert_close(k.swiglu(gu.cuda()).float().cpu(), ref.to(dtype).float(), **tol(dtype))
    torch.testing.assert_close(k.swiglu(gu.cuda()).float().cpu(), plain.swiglu(gu, dtype), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_gather(dtype):
    k = kern(dtype)
    table = rand((503, 100), dtype, 1)
    ids = torch.tensor([0, 502, 7, 7, 250], dtype=torch.int32)
    got = k.embedding(table.cuda(), ids.cuda())
    assert torch.equal(got.cpu(), torch.nn.functional.embedding(ids.long(), table))
    rows = torch.tensor([4, 0, 2], dtype=torch.int32)
    assert torch.equal(k.gather_rows(got, rows.cuda()).cpu(), got.cpu()[rows.long()])


@pytest.mark.parametrize("dtype", DTYPES)
def test_argmax_vectors(dtype):
    # The reference's vectors: ties, NaN, +-inf (python/tests/test_qwen3_kernel_contracts.py:525-539).
    k = kern(dtype)
    rows = torch.tensor([[-3.0, 7.0, 7.0, 2.0], [float("nan"), 5.0, float("nan"), 1.0],
                         [float("-inf"), float("inf"), 4.0, float("inf")]]).to(dtype)
    assert k.sample(rows.cuda()).cpu().tolist() == [1, 0, 1] == [plain.argmax_token(r) for r in rows]
    big = rand((3, 5003), dtype, 2)
    assert k.sample(big.cuda()).cpu().tolist() == torch.argmax(big.float(), dim=1).tolist()


@pytest.mark.parametrize("dtype", DTYPES)
def test_temperature_sampling(dtype):
    k = kern(dtype)
    V = 1003
    logits = rand((4, V), dtype, 3, 2.0)
    temps = torch.tensor([0.7, 1.3, 0.0, 0.7])
    u = torch.tensor([0.25, 0.9, 0.5, 0.25])
    got = k.sample(logits.cuda(), temps.cuda(), u.cuda()).cpu().tolist()
    for r in range(4):
        if temps[r] == 0:
            assert got[r] == int(torch.argmax(logits[r].float()))
            continue
        p = torch.softmax(logits[r].double() / temps[r].double(), dim=0)
        cdf = torch.cumsum(p, dim=0)
        # The drawn token's CDF interval contains u, up to float32 rounding of the running sums.
        lo = cdf[got[r] - 1] if got[r] > 0 else 0.0
        assert lo - 1e-4 <= u[r] <= cdf[got[r]] + 1e-4
    # Independent of the companions in the batch.
    assert k.sample(logits[3:4].cuda(), temps[3:4].cuda(), u[3:4].cuda()).item() == got[3]
    assert k.sample(logits[1:2].cuda(), temps[1:2].cuda(), u[1:2].cuda()).item() == got[1]
    # Temperature -> 0 is greedy; u near 1 stays inside the vocabulary.
    tiny = k.sample(logits.cuda(), torch.full((4,), 1e-4).cuda(), u.cuda()).cpu().tolist()
    assert tiny == torch.argmax(logits.float(), dim=1).tolist()
    edge = k.sample(logits.cuda(), torch.ones(4).cuda(), torch.full((4,), 1 - 2 ** -24).cuda()).cpu()
    assert ((edge >= 0) & (edge < V)).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_random_fill_matches_host(dtype):
    from vosti_amd.weights.random_init import _init_params, random_tensor_cpu, tensor_seed
    k = kern(dtype)
    for init, shape in ((("normal", 0.02), (37, 101)), (("uniform", 0.9, 1.1), (1000,))):
        host = random_tensor_cpu(5, "some.name", shape, init).to(dtype)
        dev = torch.empty(shape, dtype=dtype, device="cuda")
        k.fill_random(dev, tensor_seed(5, "some.name"), *_init_params(init))
        assert torch.equal(dev.cpu(), host)
    big = random_tensor_cpu(1, "w", (200000,), ("normal", 0.02))
    assert abs(big.std().item() - 0.02) < 3e-4 and abs(big.mean().item()) < 2e-4


# ------------------------------------------------------------------ qkv_post
def paged_layout(n_tokens, P, n_pages, seed):
    """A shuffled assignment of logical pages to physical ones."""
    g = torch.Generator().manual_seed(seed)
    need = -(-n_tokens // P)
    return torch.randperm(n_pages, generator=g)[:need].tolist()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,P,rot", [(4, 2, 16, 16, 16), (8, 2, 32, 8, 32), (3, 1, 80, 32, 40), (2, 2, 128, 64, 128)])
def test_qkv_post(dtype, nq, nkv, d, P, rot):
    k = kern(dtype)
    T, eps, max_pos, theta = 21, 1e-5, 64, 1e4
    qkv = rand((T, (nq + 2 * nkv) * d), dtype, 1)
    qw, kw = (1 + 0.1 * rand((d,), torch.float32, 2)).to(dtype), (1 + 0.1 * rand((d,), torch.float32, 3)).to(dtype)
    positions = torch.arange(5, 5 + T, dtype=torch.int32)
    inv = (1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.int64).float() / rot))).cuda()
    cos, sin = k.rope_tables(inv, max_pos)
    pcos, psin = plain.rope_tables(max_pos, rot, theta, dtype)
    torch.testing.assert_close(cos.float().cpu(), pcos, rtol=1e-5, atol=1e-5 if dtype == torch.float32 else 1e-2)
    n_pages = 9
    pages = paged_layout(5 + T, P, n_pages, 4)
    slots = torch.tensor([pages[p // P] * P + p % P for p in positions.tolist()], dtype=torch.int32)
    slots[3] = -1   # writes nothing
    kc = torch.full((n_pages, nkv, P, d), 7.0, dtype=dtype).cuda()
    vc = torch.full((n_pages, nkv, d, P), 7.0, dtype=dtype).cuda()
    q = k.qkv_post(qkv.cuda(), nq=nq, nkv=nkv, d=d, q_out=None, k_cache=kc, v_cache=vc, page_size=P, q_w=qw.cuda(),
                   k_w=kw.cuda(), eps=eps, cos=cos, sin=sin, positions=positions.cuda(), slots=slots.cuda())
    x = qkv.view(T, nq + 2 * nkv, d)
    ref_q = plain.apply_rope(plain.head_rms_norm(x[:, :nq], qw, eps, dtype), pcos, psin, positions, dtype)
    ref_k = plain.apply_rope(plain.head_rms_norm(x[:, nq:nq + nkv], kw, eps, dtype), pcos, psin, positions, dtype)
    torch.testing.assert_close(q.float().cpu(), ref_q, **tol(dtype))
    kc, vc = kc.cpu(), vc.cpu()
    written = torch.zeros(n_pages * P, dtype=torch.bool)
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        written[s] = True
        torch.testing.assert_close(kc[s // P, :, s % P, :].float(), ref_k[t], **tol(dtype))
        assert torch.equal(vc[s // P, :, :, s % P], x[t, nq + nkv:]), "a stored value row is the input row, bytewise"
    # Unwritten slots are unchanged.
    untouched_k = kc.permute(0, 2, 1, 3).reshape(n_pages * P, nkv, d)[~written]
    assert (untouched_k == 7.0).all()
    untouched_v = vc.permute(0, 3, 1, 2).reshape(n_pages * P, nkv, d)[~written]
    assert (untouched_v == 7.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,P", [(4, 2, 64, 16), (8, 2, 128, 64), (2, 1, 256, 8), (3, 3, 128, 32)])
def test_cache_store_of_a_long_step(dtype, nq, nkv, d, P):
    """A step of many tokens takes other launch shapes than a step of few (all heads of a token per workgroup).
    The rows here are decoded tokens with scattered slots, a portion that begins at a page's first place but at
    row 5 of the step, a portion that begins in the middle of a page, rows that store nothing, and a short tail:
    both caches must hold exactly what storing the rows nine at a time leaves, every value row is the input row
    bytewise, and nothing else is touched."""
    k = kern(dtype)
    n_pages, eps = 40, 1e-6
    g = torch.Generator().manual_seed(5)
    perm = torch.randperm(n_pages, generator=g).tolist()
    slots = [perm[0] * P + 3, perm[1] * P + P - 1, -1, perm[2] * P, perm[3] * P + 5]            # decoded tokens
    run = lambda page_list, first, n: [page_list[(first + i) // P] * P + (first + i) % P for i in range(n)]
    slots += run(perm[4:16], 0, 77)                    # begins at a page's first place, at row 5
    slots += [-1, -1, -1]
    slots += run(perm[16:26], 13, 50)                  # begins inside a page
    slots += run(perm[26:30], 8, 11)                   # an aligned beginning, too short for a second run
    slots[40] = -1                                     # a hole inside a run
    T = len(slots)
    assert T >= 64 and len(set(x for x in slots if x >= 0)) == len([x for x in slots if x >= 0])
    qkv = rand((T, (nq + 2 * nkv) * d), dtype, 1)
    qw, kw = (1 + 0.1 * rand((d,), torch.float32, 2)).to(dtype), (1 + 0.1 * rand((d,), torch.float32, 3)).to(dtype)
    positions = torch.arange(T, dtype=torch.int32)
    inv = (1.0 / (1e4 ** (torch.arange(0, d, 2, dtype=torch.int64).float() / d))).cuda()
    cos, sin = k.rope_tables(inv, T + 1)
    st = torch.tensor(slots, dtype=torch.int32)

    def store(rows):
        kc = torch.full((n_pages, nkv, P, d), 7.0, dtype=dtype).cuda()
        vc = torch.full((n_pages, nkv, d, P), 7.0, dtype=dtype).cuda()
        qs = [k.qkv_post(qkv[a:b].cuda(), nq=nq, nkv=nkv, d=d, q_out=None, k_cache=kc, v_cache=vc, page_size=P, q_w=qw.cuda(), k_w=kw.cuda(),
                         eps=eps, cos=cos, sin=sin, positions=positions[a:b].cuda(), slots=st[a:b].cuda()) for a, b in rows]
        return torch.cat(qs).cpu(), kc.cpu(), vc.cpu()

    q_all, kc_all, vc_all = store([(0, T)])
    q_one, kc_one, vc_one = store([(t, min(t + 9, T)) for t in range(0, T, 9)])      # nine rows a call: the launch shape of few tokens
    assert torch.equal(q_all, q_one) and torch.equal(kc_all, kc_one) and torch.equal(vc_all, vc_one)
    x = qkv.view(T, nq + 2 * nkv, d)
    written = torch.zeros(n_pages * P, dtype=torch.bool)
    for t, s_ in enumerate(slots):
        if s_ >= 0:
            written[s_] = True
            assert torch.equal(vc_all[s_ // P, :, :, s_ % P], x[t, nq + nkv:]), (t, s_)
    assert (vc_all.permute(0, 3, 1, 2).reshape(n_pages * P, nkv, d)[~written] == 7.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_invariants(dtype):
    """Position 0 is the identity; a rotation keeps each pair's norm; the product of a
    rotated q and k depends on the distance of their positions only (float32)."""
    k = kern(dtype)
    d, theta, max_pos = 32, 1e4, 128
    inv = (1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.int64).float() / d))).cuda()
    cos, sin = k.rope_tables(inv, max_pos)

    def rot(x, pos):
        T = x.shape[0]
        return k.qkv_post(x.view(T, -1), nq=x.shape[1], nkv=0, d=d, q_out=None, k_cache=None, v_cache=None, page_size=0,
                          q_w=None, k_w=None, eps=0.0, cos=cos, sin=sin,
                          positions=torch.tensor(pos, dtype=torch.int32).cuda(), slots=None)
    x = rand((3, 2, d), dtype, 1).cuda()
    assert torch.equal(rot(x, [0, 0, 0]), x)
    y = rot(x, [3, 17, 90]).float()
    xf = x.float()
    torch.testing.assert_close(y[..., :16] ** 2 + y[..., 16:] ** 2, xf[..., :16] ** 2 + xf[..., 16:] ** 2, **tol(dtype))
    if dtype == torch.float32:
        q, kk = rand((1, 1, d), dtype, 2).cuda(), rand((1, 1, d), dtype, 3).cuda()
        dots = [(rot(q, [p + 9]) * rot(kk, [p])).sum().item() for p in (0, 5, 40, 100)]
        assert max(dots) - min(dots) < 1e-4
        # A wrong sign or pairing fails this: the half-rotation form x*cos + rotate_half(x)*sin.
        pos = [11]
        c, s = cos[11].float(), sin[11].float()
        x1, x2 = q[0, 0, :16], q[0, 0, 16:]
        want = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s])
        torch.testing.assert_close(rot(q, pos)[0, 0], want, rtol=1e-6, atol=1e-6)


# ----------------------------------------------------------------- attention
def build_cache(kk, vv, P, n_pages, seed, dtype, poison=None):
    """kk, vv: lists per sequence of [len, nkv, d].  Returns caches, block table and k_len."""
    nkv, d = kk[0].shape[1:]
    fill = 0.0 if poison is None else poison
    kc = torch.full((n_pages, nkv, P, d), fill, dtype=dtype)
    vc = torch.full((n_pages, nkv, d, P), fill, dtype=dtype)
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages, generator=g).tolist()
    width = max(-(-k.shape[0] // P) for k in kk)
    table = torch.full((len(kk), width + 1), perm[-1], dtype=torch.int32)   # padded entries: a poisoned page
    for s, (k, v) in enumerate(zip(kk, vv)):
        for j in range(-(-k.shape[0] // P)):
            page = perm.pop(0)
            table[s, j] = page
            n = min(P, k.shape[0] - j * P)
            kc[page, :, :n, :] = k[j * P:j * P + n].permute(1, 0, 2)
            vc[page, :, :, :n] = v[j * P:j * P + n].permute(1, 2, 0)
    return kc, vc, table


def run_attention(k, q_list, kk, vv, P, dtype, window=0, poison=None, decode_split=None, seed=0, prompt_mode=0, decode_mode=1):
    n_pages = sum(-(-x.shape[0] // P) for x in kk) + 3
    kc, vc, table = build_cache(kk, vv, P, n_pages, seed, dtype, poison)
    q = torch.cat(q_list).cuda()
    q_lens = [x.shape[0] for x in q_list]
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    k_len = torch.tensor([x.shape[0] for x in kk], dtype=torch.int32)
    out = torch.zeros_like(q)
    pre = [(s, o) for s, n in enumerate(q_lens) if n > 1 for o in range(0, n, ATTN_ITEM_ROWS)]
    dec = [(s, 0) for s, n in enumerate(q_lens) if n == 1]
    d = q.shape[2]
    args = (q, kc.cuda(), vc.cuda(), table.cuda(), cu.cuda(), k_len.cuda())
    kw = dict(scale=d ** -0.5, window=window, max_k_len=int(k_len.max()), out=out)
    if pre:
        k.paged_attention(*args, torch.tensor(pre, dtype=torch.int32).cuda(), mode=prompt_mode, **kw)
    if dec:
        items = torch.tensor(dec, dtype=torch.int32).cuda()
        nseg = -(-int(k_len.max()) // 256) + (1 if decode_split else 0)    # more segments than needed are harmless
        scratch = torch.full((k.attn_scratch_floats(len(dec), q.shape[1], d, nseg),), float("nan"), device="cuda")    # by decoded token, not by row of the step
        k.paged_attention(*args, items, mode=decode_mode, nseg=nseg, scratch=scratch, **kw)
    return out.cpu()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,P", [(4, 2, 16, 16), (8, 2, 32, 8), (6, 1, 80, 32), (4, 4, 128, 64), (20, 1, 48, 16)])
def test_attention_against_plain(dtype, nq, nkv, d, P):
    """Lengths straddling pages and tiles (the reference's self-test uses 63/64/65/129 against
    255/256/257/321: kernels/triton_kernels/fattn_paged.py:893-924), decode rows beside prompt rows,
    a shuffled page order, and NaN in every unused page, tail and padded table entry."""
    k = kern(dtype)
    shapes = [(63, 255), (64, 256), (65, 257), (129, 321), (1, 7), (1, 300), (3, 7), (1, 1), (2, 64), (17, 17)]
    q_list, kk, vv = [], [], []
    for i, (ql, kl) in enumerate(shapes):
        q_list.append(rand((ql, nq, d), dtype, 10 + i))
        kk.append(rand((kl, nkv, d), dtype, 30 + i))
        vv.append(rand((kl, nkv, d), dtype, 50 + i))
    got = run_attention(k, q_list, kk, vv, P, dtype, poison=float("nan"))
    off = 0
    for q, kx, vx in zip(q_list, kk, vv):
        ref = plain.attention(q, kx, vx, d ** -0.5, dtype)
        torch.testing.assert_close(got[off:off + q.shape[0]].float(), ref, **tol(dtype))
        off += q.shape[0]
    # Poison changes nothing bitwise, nor does another page order or a wider segment grid.
    clean = run_attention(k, q_list, kk, vv, P, dtype, poison=None, decode_split=True, seed=5)
    assert torch.equal(clean, got)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,P,window", [(4, 1, 128, 64, 0), (6, 2, 64, 128, 0), (2, 2, 256, 64, 0), (3, 1, 128, 256, 0),
                                               (4, 2, 128, 64, 150), (2, 1, 64, 64, 64), (8, 2, 64, 64, 333)])
def test_attention_prompt_kernels_agree(dtype, nq, nkv, d, P, window):
    """Prompt rows through the kernel that shares key tiles in LDS (these head and page sizes), through
    the kernel for every shape, and as decoded tokens: the same bits, and the plain result.  Portions
    of one to a few hundred rows after contexts that end inside tiles, segments and pages; NaN in every
    unused page and tail."""
    k = kern(dtype)
    if dtype == torch.float32 and d == 256:
        assert not k.lib.vk_attn_prefill_shares_tiles(d, P)
    else:
        assert k.lib.vk_attn_prefill_shares_tiles(d, P)
    shapes = [(300, 300), (129, 641), (2, 64), (33, 289), (128, 128), (97, 1000), (31, 95), (64, 576)]
    q_list, kk, vv = [], [], []
    for i, (ql, kl) in enumerate(shapes):
        q_list.append(rand((ql, nq, d), dtype, 10 + i))
        kk.append(rand((kl, nkv, d), dtype, 30 + i))
        vv.append(rand((kl, nkv, d), dtype, 50 + i))
    got = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"))
    for mode in (2, 6, 8, 9):  # the kernel for every shape, and shared tiles with four waves, eight, and four with one buffer
        if mode != 2 and not k.lib.vk_attn_prefill_shares_tiles(d, P):
            continue
        other = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"), seed=3, prompt_mode=mode)
        assert torch.equal(got, other), mode
    off = 0
    for q, kx, vx in zip(q_list, kk, vv):
        ref = plain.attention(q, kx, vx, d ** -0.5, dtype, window=window)
        torch.testing.assert_close(got[off:off + q.shape[0]].float(), ref, **tol(dtype))
        off += q.shape[0]
    # The last rows of two sequences as decoded tokens.
    for i in (1, 5):
        q, kx, vx = q_list[i], kk[i], vv[i]
        start = sum(x.shape[0] for x in q_list[:i])
        one = run_attention(k, [q[-1:]], [kx], [vx], P, dtype, window=window)
        assert torch.equal(one[0], got[start + q.shape[0] - 1])


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_many_decoded_tokens(dtype):
    """The decode kernels: a wave per segment that asks for a tile's fragments when it needs them, with few waves
    (keys and values asked for together) and with more than a thousand (values later), a wave per segment with the
    next tile's fragments in flight, and two waves per segment: the plain result and the same bits, with and
    without a window, for groups of 1 and 20 q heads."""
    k = kern(dtype)
    P = 16
    for nq, nkv, d, window in ((8, 8, 64, 0), (8, 8, 64, 300), (20, 1, 48, 0)):
        lens = [2100 - 83 * i for i in range(24)]
        q_list = [rand((1, nq, d), dtype, 10 + i) for i in range(24)]
        kk = [rand((n, nkv, d), dtype, 40 + i) for i, n in enumerate(lens)]
        vv = [rand((n, nkv, d), dtype, 70 + i) for i, n in enumerate(lens)]
        got = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"), decode_mode=4)
        whole = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"), seed=4, decode_mode=3)
        by_wave = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"), seed=5, decode_mode=5)
        by_pair = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"), seed=6, decode_mode=7)
        assert torch.equal(whole, got) and torch.equal(by_wave, got) and torch.equal(by_pair, got)
        for i in (0, 11, 23):
            ref = plain.attention(q_list[i], kk[i], vv[i], d ** -0.5, dtype, window=window)
            torch.testing.assert_close(got[i:i + 1].float(), ref, **tol(dtype))
            alone = run_attention(k, q_list[i:i + 1], kk[i:i + 1], vv[i:i + 1], P, dtype, window=window)
            assert torch.equal(alone[0], got[i])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,P,window", [(16, 2, 128, 64, 0), (8, 1, 128, 128, 700), (3, 1, 64, 64, 0), (40, 2, 256, 64, 0),
                                               (4, 2, 80, 64, 130)])
def test_attention_decode_kernels_agree(dtype, nq, nkv, d, P, window):
    """Decoded tokens after contexts that end at every place of a tile, a segment and a page, through
    the kernel that asks for a tile's fragments when it needs them, the one with the next tile's fragments
    in flight and the one with two waves per segment (head sizes and pages they know at compile time, and one
    they do not): the same bits, and the plain result."""
    k = kern(dtype)
    lens = [1, 2, 63, 64, 65, 255, 256, 257, 320, 511, 512, 513, 1023, 1024, 1025, 1300, 1793, 2047, 2048, 2049]
    q_list = [rand((1, nq, d), dtype, 10 + i) for i in range(len(lens))]
    kk = [rand((n, nkv, d), dtype, 40 + i) for i, n in enumerate(lens)]
    vv = [rand((n, nkv, d), dtype, 70 + i) for i, n in enumerate(lens)]
    got = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"), decode_mode=4)
    by_wave = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"), seed=5, decode_mode=5)
    assert torch.equal(by_wave, got)
    # Two waves a segment: segments of one, two, three and four tiles, whole and cut by the context's end or the window.
    by_pair = run_attention(k, q_list, kk, vv, P, dtype, window=window, poison=float("nan"), seed=6, decode_mode=7)
    assert torch.equal(by_pair, got)
    for i in range(len(lens)):
        ref = plain.attention(q_list[i], kk[i], vv[i], d ** -0.5, dtype, window=window)
        torch.testing.assert_close(by_wave[i:i + 1].float(), ref, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_long_context(dtype):
    """20,000 keys: the last 130 rows as a prompt portion and the last row as a decoded token, against
    the plain result; and a key that outweighs all others at the start, the middle and the end."""
    k = kern(dtype)
    nq, nkv, d, P, L, n = 4, 1, 128, 64, 20000, 130
    q, kx, vx = rand((n, nq, d), dtype, 1), rand((L, nkv, d), dtype, 2), rand((L, nkv, d), dtype, 3)
    got = run_attention(k, [q], [kx], [vx], P, dtype)
    ref = plain.attention(q, kx, vx, d ** -0.5, dtype)
    torch.testing.assert_close(got.float(), ref, **tol(dtype))
    one = run_attention(k, [q[-1:]], [kx], [vx], P, dtype)
    assert torch.equal(one[0], got[-1])
    for far in (0, 9999, L - 1):
        q2, k2 = q[-1:].clone() * 0.1, kx.clone() * 0.1
        q2[:, :, 0] = 40.0
        k2[far, :, 0] = 40.0
        out = run_attention(k, [q2], [k2], [vx], P, dtype)
        torch.testing.assert_close(out[0].float(), vx[far].float().repeat_interleave(nq, dim=0), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_key_in_prompt_rows(dtype):
    """A key that outweighs all others, seen from the rows of a late portion of a prompt: every row at
    or after it must return its value, through the kernel that shares tiles and the other one.  Then
    with a window that still holds the key for the first rows of the portion only."""
    k = kern(dtype)
    nq, nkv, d, P, L, n = 4, 2, 64, 64, 900, 200
    for far in (0, 63, 64, 255, 256, 699, 700, 764, 899):
        q = rand((n, nq, d), dtype, 1) * 0.1
        kx, vx = rand((L, nkv, d), dtype, 2) * 0.1, rand((L, nkv, d), dtype, 3)
        q[:, :, 0] = 40.0
        kx[far, :, 0] = 40.0
        want = vx[far].float().repeat_interleave(nq // nkv, dim=0)
        for mode in (0, 2, 6, 8, 9):   # by shape, the kernel for every shape, shared tiles with four waves, eight, four and one buffer
            got = run_attention(k, [q], [kx], [vx], P, dtype, prompt_mode=mode)
            first = max(0, far - (L - n))          # the first row of the portion that sees the key
            torch.testing.assert_close(got[first:].float(), want.expand(n - first, -1, -1), **tol(dtype))
            if first:
                assert (got[:first].float() - want).abs().max() > 0.1
        if far >= L - n:
            continue
        w = L - n - far + 50                        # rows 0..49 of the portion still see the key
        got = run_attention(k, [q], [kx], [vx], P, dtype, window=w)
        torch.testing.assert_close(got[:50].float(), want.expand(50, -1, -1), **tol(dtype))
        assert (got[50:].float() - want).abs().max() > 0.1


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_cutting_is_bitwise_invisible(dtype):
    """A row's result depends on its own query and its keys only: the same position computed as a
    prompt row, as a row of a shorter portion, and as a decoded token gives the same bits."""
    k = kern(dtype)
    nq, nkv, d, P, L = 8, 2, 64, 16, 600
    q, kx, vx = rand((L, nq, d), dtype, 1), rand((L, nkv, d), dtype, 2), rand((L, nkv, d), dtype, 3)
    whole = run_attention(k, [q], [kx], [vx], P, dtype)
    for start, n in ((L - 1, 1), (300, 1), (255, 2), (250, 37), (0, 1), (511, 5)):
        part = run_attention(k, [q[start:start + n]], [kx[:start + n]], [vx[:start + n]], P, dtype, decode_split=(n == 1))
        assert torch.equal(part, whole[start:start + n]), (start, n)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_key_and_window(dtype):
    """One key among hundreds is made to stand out, so that a kernel that loses a far key, a page or
    a window's edge shows: the output must be that key's value.  Then a window that ends just before
    or just at that key."""
    k = kern(dtype)
    nq, nkv, d, P, L = 4, 2, 32, 8, 700
    for far in (0, 7, 8, 255, 256, 511, 640):
        q = rand((1, nq, d), dtype, 1) * 0.1
        kx, vx = rand((L, nkv, d), dtype, 2) * 0.1, rand((L, nkv, d), dtype, 3)
        q[0, :, 0] = 40.0
        kx[far, :, 0] = 40.0       # score 1600 * scale: everything else vanishes
        got = run_attention(k, [q], [kx], [vx], P, dtype, decode_split=True)
        want = vx[far].float().repeat_interleave(nq // nkv, dim=0)
        torch.testing.assert_close(got[0].float(), want, **tol(dtype))
        # Window: position L-1 sees keys L-window .. L-1.
        inside = run_attention(k, [q], [kx], [vx], P, dtype, window=L - far)
        torch.testing.assert_close(inside[0].float(), want, **tol(dtype))
        if far < L - 1:
            outside = run_attention(k, [q], [kx], [vx], P, dtype, window=L - far - 1)
            ref = plain.attention(q, kx, vx, d ** -0.5, dtype, window=L - far - 1)
            torch.testing.assert_close(outside.float(), ref, **tol(dtype))
            assert not torch.allclose(outside[0].float(), want, atol=0.05)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_special_cases(dtype):
    """One head without mask (a single decoded row over all keys) is the library softmax."""
    k = kern(dtype)
    d, L = 64, 200
    q, kx, vx = rand((1, 1, d), dtype, 1), rand((L, 1, d), dtype, 2), rand((L, 1, d), dtype, 3)
    got = run_attention(k, [q], [kx], [vx], 16, dtype)
    p = torch.softmax((kx[:, 0].float() @ q[0, 0].float()) * d ** -0.5, dim=0)
    torch.testing.assert_close(got[0, 0].float(), p @ vx[:, 0].float(), **tol(dtype))
    # q_len == k_len: plain causal attention through the library routine.
    q = rand((50, 2, d), dtype, 4)
    kx, vx = rand((50, 2, d), dtype, 5), rand((50, 2, d), dtype, 6)
    got = run_attention(k, [q], [kx], [vx], 8, dtype)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float().transpose(0, 1), kx.float().transpose(0, 1),
                                                           vx.float().transpose(0, 1), is_causal=True).transpose(0, 1)
    torch.testing.assert_close(got.float(), ref, **tol(dtype))


def test_attention_refuses_bad_sizes():
    from vosti_amd.kernels.ops import KernelError
    k = kern(torch.float32)
    q = torch.zeros(1, 2, 24, device="cuda")
    kc, vc = torch.zeros(2, 1, 8, 24, device="cuda"), torch.zeros(2, 1, 24, 8, device="cuda")
    i32 = lambda *v: torch.tensor(v, dtype=torch.int32, device="cuda")
    with pytest.raises(KernelError, match="head size"):
        k.paged_attention(q, kc, vc, i32(0, 1).view(1, 2), i32(0, 1), i32(1), i32(0, 0).view(1, 2), mode=1, scale=1.0,
                          max_k_len=1, nseg=1, scratch=torch.zeros(64, device="cuda"))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,K", [(8, 100, 1024), (16, 256, 4096), (1, 33, 512), (5, 48, 96), (20, 64, 1024),
                                   (100, 100, 1024), (300, 256, 2048), (129, 70, 192), (130, 64, 96), (40, 8200, 128),
                                   (8, 100, 5120), (16, 48, 8192), (3, 64, 4608), (32, 4100, 4096), (17, 33, 512),
                                   (64, 200, 1024), (33, 64, 5120), (48, 8200, 512), (20, 130, 4608), (200, 4200, 128), (515, 4500, 64),
                                   (40, 16384, 512), (8, 4200, 2560), (2, 100, 3072), (16, 300, 6144), (5, 64, 5632), (11, 72, 7168),
                                   (9, 40, 2048)])
def test_gemm_swiglu_fused_equals_separate(dtype, M, I, K):
    """The gate/up projection with the activation folded in (the streaming kernel for few rows, the
    pipelined tile kernel for many, the kernel that shares activations through LDS between them) gives
    the bits of the two separate kernels; up to 16 rows the streaming kernel has as many waves a workgroup
    as K has chunks where that is 2, 4, 5, 6, 10 or 12 (K of 1024, 2048, 2560, 3072, 5120 and 5632, 6144), else
    eight; (5, 48, 96), (20, 64, 1024)... with K no multiple of 512 and
    (130, 64, 96) fall back to them.  Between 17 and 64 rows a workgroup takes two, three or four gate
    tiles, whichever fills the compute units best: (64, 200, 1024), (48, 8200, 512) and (40, 16384, 512)."""
    k = kern(dtype)
    a, w = rand((M, K), dtype, 1).cuda(), rand((2 * I, K), dtype, 2, K ** -0.5).cuda()    # projections of order 1
    got = k.gemm_swiglu(a, w)
    gu = k.gemm(a, w, kernel=2)
    assert torch.equal(got, k.swiglu(gu))
    # Each of the two roundings against its plain function on the same input: the projection, then the
    # activation of the projection's own output (a flip of the first carried through the second is
    # several steps of the type).
    torch.testing.assert_close(gu.float().cpu(), plain.linear(a.cpu(), w.cpu(), dtype), **tol(dtype))
    torch.testing.assert_close(got.float().cpu(), plain.swiglu(gu.cpu(), dtype), **tol(dtype))


def test_pull_reads_and_keeps_nothing():
    """The measurements' yardstick: reads a buffer of any length once (the tail of the last 16 KB included) and
    writes nothing."""
    from vosti_amd.kernels.ops import KernelError
    k = kern(torch.bfloat16)
    sink = torch.full((1,), 7, dtype=torch.int32, device="cuda")
    for n in (8, 8200, 1 << 20, (1 << 20) + 24):
        t = torch.randn(n, device="cuda").to(torch.bfloat16)
        before = t.clone()
        k.pull(t, sink)
        torch.cuda.synchronize()
        assert torch.equal(t, before) and sink.item() == 7
    with pytest.raises(KernelError, match="contiguous"):
        k.pull(torch.zeros(8, 8, device="cuda", dtype=torch.bfloat16)[:, :4], sink)


def test_attention_rounds_probabilities_as_the_reference_does():
    """bfloat16: P is rounded to the element type for P.V while the normaliser sums the unrounded P
    (kernels/triton_kernels/fattn_paged.py:236-244).  On inputs where the rounding errors add up the
    kernels agree with that and with neither of the two other ways of rounding, for prompt rows and
    for decoded rows."""
    from test_plain_cpu import attention_variant, rounding_probe
    dtype = torch.bfloat16
    k = kern(dtype)
    q, kk, v = rounding_probe()
    T, d = q.shape
    q3, k3, v3 = (t.to(dtype)[:, None, :] for t in (q, kk, v))
    frac = lambda a, b: (a != b).float().mean().item()
    variants = {how: attention_variant(q, kk, v, 1.0, how) for how in ("reference", "unrounded", "both")}

    def run(q_rows, q_list_k):
        n_pages = 4
        kc, vc, table = build_cache([k3], [v3], 16, n_pages, 0, dtype, None)
        out = torch.zeros(len(q_rows), 1, d, dtype=dtype, device="cuda")
        cu = torch.tensor([0, len(q_rows)], dtype=torch.int32).cuda()
        klen = torch.tensor([q_list_k], dtype=torch.int32).cuda()
        args = (q3[q_rows].contiguous().cuda(), kc.cuda(), vc.cuda(), table.cuda(), cu, klen)
        if len(q_rows) > 1:
            k.paged_attention(*args, torch.tensor([[0, 0]], dtype=torch.int32).cuda(), mode=0, scale=1.0, max_k_len=q_list_k, out=out)
        else:
            scratch = torch.empty(k.attn_scratch_floats(1, 1, d, 1), device="cuda")
            k.paged_attention(*args, torch.tensor([[0, 0]], dtype=torch.int32).cuda(), mode=1, scale=1.0, max_k_len=q_list_k,
                              nseg=1, scratch=scratch, out=out)
        return out[:, 0].float().cpu()

    prompt_rows = run(list(range(T)), T)
    decoded = torch.cat([run([r], r + 1) for r in range(1, T)])
    for got, sl in ((prompt_rows, slice(0, T)), (decoded, slice(1, T))):
        assert frac(got, variants["reference"][sl]) < 0.01
        assert frac(got, variants["unrounded"][sl]) > 0.2 and frac(got, variants["both"][sl]) > 0.2
