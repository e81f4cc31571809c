"""Where bfloat16 values are rounded inside the fused kernels.

A comparison within one step of the type cannot tell a kernel that rounds where the reference rounds from one
that rounds a step earlier or later: both land within a step.  These tests count exact matches instead.  For
each fused kernel the reference's order of roundings and the plausible other one are written out on the CPU;
the inputs are chosen so that the two differ in a good part of the outputs (checked first, on the CPU), and
the kernel must give the reference's values nearly everywhere (a sum taken in another order flips a rare
element) and the other variant's in visibly fewer places."""
import pytest
import torch

import plain_qwen3 as plain
from test_kernels_gpu import kern, rand

pytestmark = pytest.mark.gpu

BF = torch.bfloat16


def bf(x):
    return x.to(BF).float()


def agree(a, b):
    return (a == b).float().mean().item()


def add_norm_variant(x, r, w, eps, how):
    """'reference': the sum x + r stays unrounded for the norm while its rounded copy becomes the residual
    (kernels/triton_kernels/rmsnorm_residual.py:87-125: `hidden` is stored rounded at :98 and used unrounded
    from :101 on).  'rounded': the norm of the rounded residual, what two separate kernels would compute."""
    h = x.float() + r.float()
    if how == "rounded":
        h = bf(h)
    var = (h * h).sum(-1, keepdim=True) / h.shape[-1]
    return bf((h * torch.rsqrt(var + eps)) * w.float())


def head_norm_rope_variant(x, w, eps, cos, sin, positions, how):
    """'reference': the head norm's output is stored in the model type (kernels/triton_kernels/qk_norm.py:85-95)
    and the rotation reads that (kernels/triton_kernels/rope.py:78-123).  'unrounded': the rotation of the
    unrounded norm, what a fused kernel that forgets the store would compute.  x: [T, heads, d]."""
    x = x.float()
    var = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    n = x * torch.rsqrt(var + eps) * w.float()
    if how == "reference":
        n = bf(n)
    half = cos.shape[1]
    c, s = cos[positions.long()][:, None, :], sin[positions.long()][:, None, :]
    x1, x2 = n[..., :half], n[..., half:2 * half]
    return bf(torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, n[..., 2 * half:]], dim=-1))


@pytest.mark.parametrize("T,H", [(24, 4096), (40, 96), (30, 100), (6, 16384), (3, 32768)])
def test_add_norm_sees_the_unrounded_sum(T, H):
    """Rows in registers (4,096), short rows, a width that no vector divides (100), rows kept in LDS (16,384 and
    32,768).  The residual is three eighths of a step of x, up or down, so that the sum is exact in 32-bit and
    its rounding always loses that much: the two variants then differ in more than a third of the outputs
    (with a random residual in a fifth)."""
    k = kern(BF)
    x = rand((T, H), BF, 1)
    step = torch.exp2(torch.floor(torch.log2(x.float().abs().clamp_min(1e-30))) - 7)
    r = (torch.where(rand((T, H), torch.float32, 2) > 0, 1.0, -1.0) * 0.375 * step).to(BF)
    w = (1 + 0.1 * rand((H,), torch.float32, 3)).to(BF)
    eps = 1e-6
    ref, other = add_norm_variant(x, r, w, eps, "reference"), add_norm_variant(x, r, w, eps, "rounded")
    assert agree(ref, other) < 0.7, "the probe does not tell the variants apart"
    for w_dev in (w.cuda(), w.float().cuda()):                 # the weight in the model type and kept in 32-bit
        res = r.clone().cuda()
        got = k.add_rmsnorm(x.cuda(), res, w_dev, eps).float().cpu()
        assert agree(got, ref) > 0.99 and agree(got, other) < 0.7, (agree(got, ref), agree(got, other))
        assert torch.equal(res.float().cpu(), bf(x.float() + r.float())), "the residual is the rounded sum"
    # A residual of x's own size: its stored sum is rounded from the exact one.
    r2 = rand((T, H), BF, 4, 0.37)
    res = r2.clone().cuda()
    got = k.add_rmsnorm(x.cuda(), res, w.cuda(), eps).float().cpu()
    assert torch.equal(res.float().cpu(), bf(x.float() + r2.float()))
    assert agree(got, add_norm_variant(x, r2, w, eps, "reference")) > 0.99 > 0.8 > agree(got, add_norm_variant(x, r2, w, eps, "rounded"))
    # The reference's own arithmetic, as the plain implementation has it.
    assert agree(plain.add_rms_norm(x, r, w, eps, BF)[0], ref) == 1.0


@pytest.mark.parametrize("nq,nkv,d", [(8, 2, 128), (4, 4, 64), (2, 1, 256), (6, 2, 80), (5, 1, 32), (3, 3, 16)])
def test_head_norm_is_rounded_before_the_rotation(nq, nkv, d):
    """Head sizes whose lanes own 16 bytes of a head (64, 128, 256) and the kernel with a wave per head (the
    others): q as returned, k as stored in the cache."""
    k = kern(BF)
    T, P, eps, theta, max_pos = 40, 16, 1e-6, 1e4, 4096
    qkv = rand((T, (nq + 2 * nkv) * d), BF, 1)
    qw, kw = (1 + 0.1 * rand((d,), torch.float32, 2)).to(BF), (1 + 0.1 * rand((d,), torch.float32, 3)).to(BF)
    positions = torch.arange(1000, 1000 + T, dtype=torch.int32)            # far from 0, where a rotation is the identity
    from vosti_amd.cache.host import rotary_inverse_frequencies
    cos, sin = k.rope_tables(torch.from_numpy(rotary_inverse_frequencies(theta, d)).cuda(), max_pos)
    pcos, psin = cos.float().cpu(), sin.float().cpu()
    x = qkv.view(T, nq + 2 * nkv, d)
    slots = torch.arange(T, dtype=torch.int32)
    kc = torch.zeros(-(-T // P), nkv, P, d, dtype=BF).cuda()
    vc = torch.zeros(-(-T // P), nkv, d, P, dtype=BF).cuda()
    q = k.qkv_post(qkv.cuda(), nq=nq, nkv=nkv, d=d, q_out=None, k_cache=kc, v_cache=vc, page_size=P, q_w=qw.cuda(), k_w=kw.cuda(),
                   eps=eps, cos=cos, sin=sin, positions=positions.cuda(), slots=slots.cuda()).float().cpu()
    stored_k = kc.cpu().permute(0, 2, 1, 3).reshape(-1, nkv, d)[:T].float()
    for got, rows, w in ((q, x[:, :nq], qw), (stored_k, x[:, nq:nq + nkv], kw)):
        ref = head_norm_rope_variant(rows, w, eps, pcos, psin, positions, "reference")
        other = head_norm_rope_variant(rows, w, eps, pcos, psin, positions, "unrounded")
        assert agree(ref, other) < 0.75, "the probe does not tell the variants apart"
        assert agree(got, ref) > 0.99 and agree(got, other) < 0.75, (agree(got, ref), agree(got, other))
        two_steps = plain.apply_rope(plain.head_rms_norm(rows, w, eps, BF), pcos, psin, positions, BF)
        assert agree(two_steps, ref) == 1.0
