"""Each part alone, built from its PartSpec through the registry, against the plain function."""
import pytest
import torch

import plain_qwen3 as plain
from vosti_amd.config import PartSpec

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    # bfloat16: one step of the type where a sum in another order lands on the neighbouring value.
    return dict(rtol=2 ** -7, atol=2 ** -8) if dtype == torch.bfloat16 else dict(rtol=2e-5, atol=2e-5)


def rand(shape, dtype, seed, scale=1.0):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def build(category, kind, dtype, **params):
    from vosti_amd.kernels import kernels_for
    from vosti_amd.parts import build_part
    return build_part(category, PartSpec(kind, params), kernels_for(dtype))


def load(part, dtype, seed=0, scale=0.1):
    """Random tensors for everything the part (and its sub-parts) declares; returns them by path."""
    from vosti_amd.models.decoder import walk_params
    tensors, per_owner = {}, {}
    for i, (path, owner, local, ps) in enumerate(walk_params(part)):
        t = rand(ps.shape, dtype, seed + i, scale) + (1.0 if ps.init[0] == "uniform" else 0.0)
        tensors[path] = t.to(dtype)
        per_owner.setdefault(id(owner), (owner, {}))[1][local] = tensors[path].cuda()
    for owner, group in per_owner.values():
        owner.load(group)
    return tensors


def step_context(kernels, starts, q_lens, page, pages_of, n_pages, window=0):
    """A StepContext for sequences whose logical pages are pages_of[s]."""
    from vosti_amd.parts import GroupTables, HostStep, StepContext
    from vosti_amd.parts.standard import Attention
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    positions = [p for s, n in zip(starts, q_lens) for p in range(s, s + n)]
    slots = [pages_of[i][p // page] * page + p % page for i, (s, n) in enumerate(zip(starts, q_lens)) for p in range(s, s + n)]
    width = max(len(p) for p in pages_of)
    table = [p + [0] * (width - len(p)) for p in pages_of]
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    k_len = [s + n for s, n in zip(starts, q_lens)]
    host = HostStep(q_lens=list(q_lens), starts=list(starts), k_lens=k_len, state_slots=list(range(len(q_lens))),
                    k_len_bound=max(k_len))
    # The arrays the attention part asks of a step, uploaded as the step function would.
    inputs = {name: i32(arr.tolist()).view(-1, 2) for name, arr in Attention._items_arrays(host).items()}
    scratch = torch.empty(1 << 20, device="cuda")
    return StepContext(kernels=kernels, num_tokens=sum(q_lens), num_seqs=len(q_lens), positions=i32(positions), cu_q=i32(cu),
                       k_len=i32(k_len), state_slots=i32(list(range(len(q_lens)))),
                       groups=[GroupTables(i32(slots), i32(table), window)], host=host, inputs=inputs,
                       workspace=lambda n: scratch)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_norm_head_swiglu(dtype):
    emb = build("embedding", "token_embedding", dtype, vocab_size=77, hidden_size=40)
    w = load(emb, dtype)
    ids = torch.tensor([0, 76, 5, 5], dtype=torch.int32)
    assert torch.equal(emb.forward(ids.cuda()).cpu(), w["weight"][ids.long()])

    norm = build("norm", "rmsnorm", dtype, size=40, eps=1e-5)
    w = load(norm, dtype)
    x, r = rand((6, 40), dtype, 5), rand((6, 40), dtype, 6)
    torch.testing.assert_close(norm.forward(x.cuda()).float().cpu(), plain.rms_norm(x, w["weight"], 1e-5, dtype), **tol(dtype))
    res = r.clone().cuda()
    got = norm.forward_add(x.cuda(), res)
    pn, pr = plain.add_rms_norm(x, r, w["weight"], 1e-5, dtype)
    torch.testing.assert_close(got.float().cpu(), pn, **tol(dtype))
    torch.testing.assert_close(res.float().cpu(), pr, **tol(dtype))

    head = build("head", "linear_head", dtype, vocab_size=77, hidden_size=40, tied=False)
    w = load(head, dtype)
    torch.testing.assert_close(head.forward(x.cuda()).float().cpu(), plain.linear(x, w["weight"], dtype), **tol(dtype))
    # A tied head is the same part: the architecture names its weight like the embedding's table.
    assert list(build("head", "linear_head", dtype, vocab_size=77, hidden_size=40, tied=True).params()) == ["weight"]

    ffn = build("feed_forward", "swiglu", dtype, hidden_size=40, intermediate_size=56)
    w = load(ffn, dtype)
    gu = torch.cat([plain.linear(x, w["gate_proj.weight"], dtype), plain.linear(x, w["up_proj.weight"], dtype)], 1)
    ref = plain.linear(plain.swiglu(gu, dtype), w["down_proj.weight"], dtype)
    torch.testing.assert_close(ffn.forward(x.cuda(), None).float().cpu(), ref, **tol(dtype))


def test_projections_with_a_workspace_give_the_same_bits():
    """With 17 to 64 rows the larger projections go through chunk sums in the step's workspace; the parts
    announce how much of it they need, and the result is what they compute without one."""
    from vosti_amd.kernels import kernels_for
    from vosti_amd.parts import HostStep
    dtype, k = torch.bfloat16, kernels_for(torch.bfloat16)
    host = HostStep(q_lens=[40], starts=[0], k_lens=[40], state_slots=[0], k_len_bound=40)
    ffn = build("feed_forward", "swiglu", dtype, hidden_size=1024, intermediate_size=8192)
    load(ffn, dtype, scale=0.03)
    assert ffn.workspace_floats(host) == k.gemm_workspace_floats(40, 1024, 8192) > 0
    x = rand((40, 1024), dtype, 3).cuda()
    ctx = step_context(k, [0], [40], 64, [[0]], 1)
    ctx.workspace = lambda n, buf=torch.full((ffn.workspace_floats(host),), float("nan"), device="cuda"): buf
    assert torch.equal(ffn.forward(x, ctx), ffn.forward(x, None))
    rope = PartSpec("rotary", {"head_dim": 128, "rotary_dim": 128, "theta": 1e4, "max_positions": 64})
    att = build("mixer", "attention", dtype, hidden_size=2048, num_heads=16, num_kv_heads=8, head_dim=128, scale=128 ** -0.5,
                position=rope)
    load(att, dtype, scale=0.03)
    assert att.workspace_floats(host) == k.gemm_workspace_floats(40, 32 * 128, 2048) > 0
    from vosti_amd.parts import PagedKV
    x = rand((40, 2048), dtype, 4).cuda()
    outs = []
    for with_workspace in (True, False):
        cache = PagedKV(torch.zeros(1, 8, 64, 128, dtype=dtype, device="cuda"), torch.zeros(1, 8, 128, 64, dtype=dtype, device="cuda"), 0, 64)
        ctx = step_context(k, [0], [40], 64, [[0]], 1)
        if not with_workspace:
            ctx.workspace = None
        outs.append(att.forward(x, ctx, cache))
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotary_part(dtype):
    rot = build("position", "rotary", dtype, head_dim=32, rotary_dim=32, theta=1e4, max_positions=64)
    q, k = rand((5, 3, 32), dtype, 1), rand((5, 1, 32), dtype, 2)
    pos = torch.tensor([0, 1, 9, 33, 63], dtype=torch.int32)
    q2, k2 = rot.apply(q.cuda(), k.cuda(), pos.cuda())
    cos, sin = plain.rope_tables(64, 32, 1e4, dtype)
    torch.testing.assert_close(q2.float().cpu(), plain.apply_rope(q, cos, sin, pos, dtype), **tol(dtype))
    torch.testing.assert_close(k2.float().cpu(), plain.apply_rope(k, cos, sin, pos, dtype), **tol(dtype))
    # The table in float32 is bitwise what the plain formula gives for the frequencies, and close for the angles.
    if dtype == torch.float32:
        torch.testing.assert_close(rot.cos.cpu(), cos, rtol=0, atol=2e-6)
    with pytest.raises(ValueError, match="rotary width"):
        build("position", "rotary", dtype, head_dim=32, rotary_dim=34, theta=1e4, max_positions=8)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,fused", [(0, True), (20, True), (0, False)])
def test_attention_part(dtype, window, fused):
    """The whole mixer: projections, head norms, rotation, store, attention, output projection; a prompt
    in two portions and then a decoded token, over shuffled pages.  fused=False puts a norm subclass in,
    so that the mixer takes its step-by-step path."""
    from vosti_amd.parts import PagedKV, register_part
    from vosti_amd.parts.standard import RMSNorm
    H, nq, nkv, d, page, eps = 48, 6, 2, 16, 8, 1e-5
    norm_kind = "rmsnorm"
    if not fused:
        @register_part("norm", "rmsnorm_twin")
        class Twin(RMSNorm):
            pass
        norm_kind = "rmsnorm_twin"
    hn = PartSpec(norm_kind, {"size": d, "eps": eps})
    att = build("mixer", "attention", dtype, hidden_size=H, num_heads=nq, num_kv_heads=nkv, head_dim=d, scale=d ** -0.5,
                window=window, q_norm=hn, k_norm=hn,
                position=PartSpec("rotary", {"head_dim": d, "rotary_dim": d, "theta": 1e4, "max_positions": 128}))
    assert att._fused == fused
    w = load(att, dtype, scale=0.2)
    T = 45
    x = rand((T, H), dtype, 9)
    # plain
    pos = torch.arange(T)
    q = plain.head_rms_norm(plain.linear(x, w["q_proj.weight"], dtype).view(T, nq, d), w["q_norm.weight"], eps, dtype)
    k = plain.head_rms_norm(plain.linear(x, w["k_proj.weight"], dtype).view(T, nkv, d), w["k_norm.weight"], eps, dtype)
    v = plain.linear(x, w["v_proj.weight"], dtype).view(T, nkv, d)
    cos, sin = plain.rope_tables(128, d, 1e4, dtype)
    q, k = plain.apply_rope(q, cos, sin, pos, dtype), plain.apply_rope(k, cos, sin, pos, dtype)
    ref = plain.linear(plain.attention(q, k, v, d ** -0.5, dtype, window=window).reshape(T, nq * d), w["o_proj.weight"], dtype)
    # engine part: pages 5, 2, 7, 0, 3, 6 hold the sequence
    pages = [5, 2, 7, 0, 3, 6]
    cache = PagedKV(torch.full((8, nkv, page, d), float("nan"), dtype=dtype, device="cuda"),
                    torch.full((8, nkv, d, page), float("nan"), dtype=dtype, device="cuda"), group=0, page_size=page)
    outs = []
    for start, n in ((0, 30), (30, 14), (44, 1)):
        ctx = step_context(att.kernels, [start], [n], page, [pages], 8, window)
        outs.append(att.forward(x[start:start + n].cuda().contiguous(), ctx, cache))
    torch.testing.assert_close(torch.cat(outs).float().cpu(), ref, **tol(dtype))
    assert att.cache_spec().window == window and att.cache_spec().num_kv_heads == nkv


@pytest.mark.parametrize("dtype", DTYPES)
def test_prenorm_block(dtype):
    """The arrangement alone, with the framework's parts inside: equal to the plain layer function on (hidden, residual)."""
    from vosti_amd.config import LayerSpec
    from vosti_amd.kernels import kernels_for
    from vosti_amd.models.decoder import _build_block
    from vosti_amd.parts import PagedKV
    H, nq, nkv, d, page, eps, I = 32, 2, 1, 16, 8, 1e-6, 48
    norm = PartSpec("rmsnorm", {"size": H, "eps": eps})
    mixer = PartSpec("attention", {"hidden_size": H, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d, "scale": 0.25})
    spec = LayerSpec("prenorm", mixer, PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}),
                     {"input": norm, "post_mixer": norm}, {})
    block = _build_block(spec, kernels_for(dtype))
    w = load(block, dtype, scale=0.2)
    T = 11
    hidden, residual = rand((T, H), dtype, 3), rand((T, H), dtype, 4)
    n1, res = plain.add_rms_norm(hidden, residual, w["norms.input.weight"], eps, dtype)
    q = plain.linear(n1, w["mixer.q_proj.weight"], dtype).view(T, nq, d)
    k = plain.linear(n1, w["mixer.k_proj.weight"], dtype).view(T, nkv, d)
    v = plain.linear(n1, w["mixer.v_proj.weight"], dtype).view(T, nkv, d)
    a = plain.linear(plain.attention(q, k, v, 0.25, dtype).reshape(T, nq * d), w["mixer.o_proj.weight"], dtype)
    n2, res = plain.add_rms_norm(a, res, w["norms.post_mixer.weight"], eps, dtype)
    gu = torch.cat([plain.linear(n2, w["feed_forward.gate_proj.weight"], dtype), plain.linear(n2, w["feed_forward.up_proj.weight"], dtype)], 1)
    ref = plain.linear(plain.swiglu(gu, dtype), w["feed_forward.down_proj.weight"], dtype)
    cache = PagedKV(torch.zeros(2, nkv, page, d, dtype=dtype, device="cuda"), torch.zeros(2, nkv, d, page, dtype=dtype, device="cuda"), 0, page)
    ctx = step_context(block.kernels, [0], [T], page, [[1, 0]], 2)
    res_dev = residual.clone().cuda()
    out, res_out = block.forward(hidden.cuda(), res_dev, ctx, cache)
    torch.testing.assert_close(out.float().cpu(), ref, **tol(dtype))
    torch.testing.assert_close(res_out.float().cpu(), res, **tol(dtype))
    with pytest.raises(ValueError, match="post_mixer"):
        _build_block(LayerSpec("prenorm", mixer, spec.feed_forward, {"input": norm}, {}), kernels_for(dtype))
    with pytest.raises(ValueError, match="no mixer part of kind"):
        _build_block(LayerSpec("prenorm", PartSpec("nope", {}), spec.feed_forward, spec.norms, {}), kernels_for(dtype))
