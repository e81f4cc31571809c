"""Pins the plain implementation by what fixes it beside the reference's text: vectors the
reference's tests hold, special cases that reduce to a library routine, and invariants, each chosen
so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""
import math

import pytest
import torch

import plain_qwen3 as plain
from conftest import TINY

F32 = torch.float32


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def test_embedding_is_the_library_lookup():
    # kernels/tests/runtime/test_embedding.py:27-32: equal to torch's embedding, tolerance 0.
    table, ids = rnd(11, 6), torch.tensor([3, 0, 10, 3])
    assert torch.equal(plain.embedding(ids, table), torch.nn.functional.embedding(ids, table))


def test_rms_norm_properties():
    x, w = rnd(5, 48, seed=1), 1 + 0.1 * rnd(48, seed=2)
    # kernels/triton_kernels/rmsnorm.py:157-161: the reference's own check.
    ref = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-6, F32), ref)
    y = plain.rms_norm(x * 37.0, torch.ones(48), 0.0, F32)
    torch.testing.assert_close(y.pow(2).mean(-1).sqrt(), torch.ones(5))          # unit RMS, scale invariant
    torch.testing.assert_close(y, plain.rms_norm(x, torch.ones(48), 0.0, F32))
    # eps sits inside the square root, added to the mean (not to the sum, not outside).
    z = torch.zeros(1, 4)
    assert torch.equal(plain.rms_norm(z, torch.ones(4), 1e-6, F32), z)
    one = torch.full((1, 4), 2.0)
    torch.testing.assert_close(plain.rms_norm(one, torch.ones(4), 5.0, F32), one / 3.0)   # 2 / sqrt(4 + 5)


def test_add_rms_norm_sees_the_unrounded_sum():
    # kernels/triton_kernels/rmsnorm_residual.py:197-202: residual_out == x + r, normed == rmsnorm(x + r).
    x, r, w = rnd(4, 32, seed=3), rnd(4, 32, seed=4), 1 + 0.1 * rnd(32, seed=5)
    n, res = plain.add_rms_norm(x, r, w, 1e-6, F32)
    assert torch.equal(res, x + r)
    torch.testing.assert_close(n, plain.rms_norm(x + r, w, 1e-6, F32))
    # In bfloat16 the stored residual is rounded but the norm is not computed from the rounded one.
    xb, rb = x.bfloat16().float() * 100, r.bfloat16().float()
    n16, res16 = plain.add_rms_norm(xb, rb, w, 1e-6, torch.bfloat16)
    assert torch.equal(res16, (xb + rb).bfloat16().float())
    exact = ((xb + rb) * torch.rsqrt((xb + rb).pow(2).mean(-1, keepdim=True) + 1e-6) * w).bfloat16().float()
    assert torch.equal(n16, exact)


def test_head_norm_is_the_row_norm_per_head():
    # kernels/triton_kernels/qk_norm.py:188-190: reshape to [T*heads, d] and apply the plain norm.
    x, w = rnd(3, 4, 16, seed=6), 1 + 0.1 * rnd(16, seed=7)
    torch.testing.assert_close(plain.head_rms_norm(x, w, 1e-5, F32),
                               plain.rms_norm(x.reshape(12, 16), w, 1e-5, F32).view(3, 4, 16))


def test_rope():
    d, theta = 16, 1e4
    cos, sin = plain.rope_tables(64, d, theta, F32)
    # The first frequency is 1, the last theta^-((d-2)/d): python/vosti_kernels/rotary.py:80-90.
    torch.testing.assert_close(cos[5, 0], torch.tensor(math.cos(5.0)))
    torch.testing.assert_close(sin[9, d // 2 - 1], torch.tensor(math.sin(9.0 * theta ** (-(d - 2) / d))))
    x = rnd(4, 2, d, seed=8)
    pos = torch.tensor([0, 3, 17, 40])
    y = plain.apply_rope(x, cos, sin, pos, F32)
    assert torch.equal(y[0], x[0])                                               # position 0 is the identity
    torch.testing.assert_close(y[..., :8] ** 2 + y[..., 8:] ** 2, x[..., :8] ** 2 + x[..., 8:] ** 2)   # pairs (j, j + d/2)
    # x*cos + rotate_half(x)*sin with rotate_half = cat(-x2, x1): python/vosti_kernels/kernels.py:472-482.
    c, s = torch.cat([cos[pos], cos[pos]], -1)[:, None], torch.cat([sin[pos], sin[pos]], -1)[:, None]
    rot_half = torch.cat([-x[..., 8:], x[..., :8]], -1)
    torch.testing.assert_close(y, x * c + rot_half * s)
    # Only distances count: shifting both positions leaves q.k unchanged.
    q, k = rnd(1, 1, d, seed=9), rnd(1, 1, d, seed=10)
    dots = [(plain.apply_rope(q, cos, sin, torch.tensor([p + 7]), F32) * plain.apply_rope(k, cos, sin, torch.tensor([p]), F32)).sum()
            for p in (0, 1, 20, 50)]
    torch.testing.assert_close(torch.stack(dots), dots[0].expand(4), rtol=1e-4, atol=1e-5)
    # ... and the sign is the one that makes it depend on (query - key), not (key - query).
    back = (plain.apply_rope(q, cos, sin, torch.tensor([3]), F32) * plain.apply_rope(k, cos, sin, torch.tensor([10]), F32)).sum()
    assert abs(back - dots[0]) > 1e-3
    # A partial rotation leaves the rest of the head alone.
    c8, s8 = plain.rope_tables(64, 8, theta, F32)
    assert torch.equal(plain.apply_rope(x, c8, s8, pos, F32)[..., 8:], x[..., 8:])
    # Tables in bfloat16 are the float32 tables rounded (rotary.py:160).
    cb, _ = plain.rope_tables(64, d, theta, torch.bfloat16)
    assert torch.equal(cb, cos.bfloat16().float())


@pytest.mark.parametrize("q_len,k_len", [(4, 4), (1, 7), (3, 7), (7, 3), (3, 0)])
def test_attention_oracle_shapes(q_len, k_len):
    # kernels/tests/runtime/test_attention_sdpa_reference.py:8-55: bottom-right aligned causal GQA against an
    # explicit softmax per row, for these five (q_len, k_len) pairs.
    nq, nkv, d = 4, 2, 8
    q, k, v = rnd(q_len, nq, d, seed=1), rnd(k_len, nkv, d, seed=2), rnd(k_len, nkv, d, seed=3)
    out = plain.attention(q, k, v, d ** -0.5, F32)
    for r in range(q_len):
        p = k_len - q_len + r
        for h in range(nq):
            if p < 0:
                assert torch.equal(out[r, h], torch.zeros(d))
                continue
            g = h // (nq // nkv)
            w = torch.softmax((k[:p + 1, g].double() @ q[r, h].double()) * d ** -0.5, 0)
            torch.testing.assert_close(out[r, h].double(), w @ v[:p + 1, g].double(), rtol=1e-5, atol=1e-6)


def test_attention_reduces_to_the_library_routine():
    nq, nkv, d, T = 6, 2, 16, 12
    q, k, v = rnd(T, nq, d, seed=4), rnd(T, nkv, d, seed=5), rnd(T, nkv, d, seed=6)
    out = plain.attention(q, k, v, d ** -0.5, F32)
    # Groups are contiguous: head h reads kv head h // (nq / nkv), i.e. repeat_interleave
    # (kernels/triton_kernels/fattn_paged.py:716-763).
    kr, vr = k.repeat_interleave(nq // nkv, dim=1), v.repeat_interleave(nq // nkv, dim=1)
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), kr.transpose(0, 1), vr.transpose(0, 1),
                                                           is_causal=True).transpose(0, 1)
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-6)
    # One head, one decoded row, no rotation or mask: a softmax over the history.
    o1 = plain.attention(q[-1:, :1], k[:, :1], v[:, :1], 1.0, F32)
    torch.testing.assert_close(o1[0, 0], torch.softmax(k[:, 0] @ q[-1, 0], 0) @ v[:, 0], rtol=1e-5, atol=1e-6)
    # Window w: position p sees keys p - w + 1 .. p.
    ow = plain.attention(q, kr, vr, d ** -0.5, F32, window=3)
    mask = torch.ones(T, T).tril().bool() & ~torch.ones(T, T).tril(-3).bool()
    refw = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), kr.transpose(0, 1), vr.transpose(0, 1),
                                                            attn_mask=mask).transpose(0, 1)
    torch.testing.assert_close(ow, refw, rtol=1e-5, atol=1e-6)


def test_swiglu_and_sampler():
    gu = rnd(3, 10, seed=7, scale=3.0)
    torch.testing.assert_close(plain.swiglu(gu, F32), torch.nn.functional.silu(gu[:, :5]) * gu[:, 5:])   # silu_mul.py:146
    # python/tests/test_qwen3_kernel_contracts.py:525-539.
    rows = torch.tensor([[-3.0, 7.0, 7.0, 2.0], [float("nan"), 5.0, float("nan"), 1.0],
                         [float("-inf"), float("inf"), 4.0, float("inf")]])
    assert [plain.argmax_token(r) for r in rows] == [1, 0, 1] and plain.argmax_token(torch.empty(0)) == 0


@pytest.fixture(scope="module")
def model_a(tiny_dirs):
    return plain.PlainQwen3(tiny_dirs["A"], F32)


def test_whole_model_is_the_textbook_pre_norm_decoder(model_a):
    """The (hidden, residual) pair of the reference is x += attn(norm(x)); x += mlp(norm(x)) in
    disguise (src/proof/model/dense_swiglu/semantics.rs:266-347).  A norm in the wrong place, a
    missing residual or a post-norm arrangement fails this."""
    m, w = model_a, model_a.w
    ids = [5, 200, 17, 17, 99, 3, 250, 0, 1]
    pos = torch.arange(len(ids))
    x = w["model.embed_tokens.weight"][torch.tensor(ids)]
    for i in range(m.L):
        p = f"model.layers.{i}."
        n = plain.rms_norm(x, w[p + "input_layernorm.weight"], m.eps, F32)
        T = len(ids)
        q = plain.head_rms_norm((n @ w[p + "self_attn.q_proj.weight"].t()).view(T, m.nq, m.d), w[p + "self_attn.q_norm.weight"], m.eps, F32)
        k = plain.head_rms_norm((n @ w[p + "self_attn.k_proj.weight"].t()).view(T, m.nkv, m.d), w[p + "self_attn.k_norm.weight"], m.eps, F32)
        v = (n @ w[p + "self_attn.v_proj.weight"].t()).view(T, m.nkv, m.d)
        q, k = plain.apply_rope(q, m.cos, m.sin, pos, F32), plain.apply_rope(k, m.cos, m.sin, pos, F32)
        a = plain.attention(q, k, v, m.d ** -0.5, F32).reshape(T, -1)
        x = x + a @ w[p + "self_attn.o_proj.weight"].t()
        n = plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], m.eps, F32)
        g, u = n @ w[p + "mlp.gate_proj.weight"].t(), n @ w[p + "mlp.up_proj.weight"].t()
        x = x + (torch.nn.functional.silu(g) * u) @ w[p + "mlp.down_proj.weight"].t()
    ref = plain.rms_norm(x, w["model.norm.weight"], m.eps, F32) @ w["model.embed_tokens.weight"].t()   # tied head
    torch.testing.assert_close(m.logits(ids), ref, rtol=1e-4, atol=1e-5)


def test_causality_and_position_dependence(model_a):
    ids = [9, 8, 7, 6, 5, 4, 3, 2]
    full = model_a.logits(ids)
    torch.testing.assert_close(model_a.logits(ids[:5]), full[:5], rtol=1e-5, atol=1e-6)     # the future is invisible
    changed = model_a.logits([1] + ids[1:])
    assert (changed[-1] - full[-1]).abs().max() > 1e-4                                     # the far past is not


def test_lm_head_on_selected_rows_equals_row_selection(model_a):
    # src/exec/dense_swiglu_model.rs:986-1017 proves exactly this; the reference's gather vector is
    # cu_q = [0, 2, 5, 6] -> rows [1, 4, 5] (python/tests/test_qwen3_kernel_contracts.py:515-520).
    hidden = torch.arange(24, dtype=F32).reshape(6, 4)
    cu = torch.tensor([0, 2, 5, 6])
    rows = cu[1:] - 1
    assert rows.tolist() == [1, 4, 5]
    wmat = rnd(7, 4, seed=11)
    assert torch.equal(plain.linear(hidden[rows], wmat, F32), plain.linear(hidden, wmat, F32)[rows])


def test_bfloat16_mode_rounds_where_the_reference_stores(tiny_dirs):
    m32, m16 = plain.PlainQwen3(tiny_dirs["B"], F32), plain.PlainQwen3(tiny_dirs["B"], torch.bfloat16)
    ids = list(range(40, 75))
    a, b = m32.logits(ids), m16.logits(ids)
    assert torch.equal(b, b.bfloat16().float())            # logits leave the model in the model type
    err = (a - b).abs().max().item()
    assert 1e-4 < err < 0.1


def test_head_norm_comes_before_the_rotation(tiny_dirs):
    """The q/k head norm is applied before the rotary encoding (src/exec/dense_swiglu_decoder.rs:207-246).
    What fixes the order beside that text: with the norm first, the vectors that are rotated do not
    depend on the position, so scores depend on distances only and the logits of a sequence do not
    change when all its positions are shifted.  With the rotation first, the norm's weights (which
    differ between the two halves of a rotated pair) scale the pair's two members differently after
    the rotation, and the invariance is lost.  The swapped model, written out here, fails it."""
    m = plain.PlainQwen3(tiny_dirs["B"], F32)
    ids = [11, 400, 7, 7, 250, 33, 1, 499, 60, 61, 62, 5]
    base = m.logits(ids)
    for shift in (1, 37, 200):
        torch.testing.assert_close(m.logits(ids, first_position=shift), base, rtol=1e-4, atol=2e-5)

    class Swapped(plain.PlainQwen3):
        def layer(self, i, hidden, residual, positions):
            real_norm, real_rope = plain.head_rms_norm, plain.apply_rope
            pending = {}

            def norm_later(x, w, eps, dt):      # remember the weight, leave x alone until after the rotation
                pending[x.shape[1]] = (w, eps)
                return x

            def rope_then_norm(x, cos, sin, pos, dt):
                w, eps = pending[x.shape[1]]
                return real_norm(real_rope(x, cos, sin, pos, dt), w, eps, dt)
            plain.head_rms_norm, plain.apply_rope = norm_later, rope_then_norm
            try:
                return super().layer(i, hidden, residual, positions)
            finally:
                plain.head_rms_norm, plain.apply_rope = real_norm, real_rope

    sw = Swapped(tiny_dirs["B"], F32)
    assert (sw.logits(ids) - base).abs().max() > 1e-3                                  # it is another model
    assert (sw.logits(ids, first_position=37) - sw.logits(ids)).abs().max() > 1e-3      # and not shift-invariant


def attention_variant(q, k, v, scale, how):
    """One head, all rows, vectorised, with the probabilities' rounding written out three ways:
    'reference': P rounded to bfloat16 for the product, normaliser from the unrounded P
    (kernels/triton_kernels/fattn_paged.py:236-244); 'unrounded': nothing rounded; 'both': the
    normaliser from the rounded P too."""
    T = q.shape[0]
    s = (q @ k.t()) * scale
    s = s.masked_fill(~torch.ones(T, T).tril().bool(), float("-inf"))
    e = torch.exp(s - s.max(-1, keepdim=True).values)
    eb = e.bfloat16().float()
    num = (e if how == "unrounded" else eb) @ v
    den = (eb if how == "both" else e).sum(-1, keepdim=True)
    return (num / den).bfloat16().float()


def rounding_probe(T=48, d=32, delta=1.046875, seed=23):
    """Inputs on which the rounding of the probabilities shows: row r sees key 0 with score 0 and keys
    1..r with score -delta each (scale 1), so every probability but one is exp(-delta) = 0.35103, which
    bfloat16 rounds up by 0.15 %; the values are positive, so the errors add up instead of cancelling.
    All inputs are exact in bfloat16."""
    q = torch.zeros(T, d)
    q[:, 0] = 1.0
    k = torch.zeros(T, d)
    k[1:, 0] = -delta
    v = (torch.rand(T, d, generator=torch.Generator().manual_seed(seed)) + 0.5).bfloat16().float()
    return q, k, v


def test_probabilities_are_rounded_before_they_meet_the_values():
    """fattn_paged.py:236-244: p is cast to the value type for the dot product, l_i sums the float32 p.
    On inputs where the rounding errors add up, the three ways of rounding give visibly different
    outputs, and the plain attention is the first."""
    q, k, v = rounding_probe()
    got = plain.attention(q[:, None], k[:, None], v[:, None], 1.0, torch.bfloat16)[:, 0]
    frac = lambda a, b: (a != b).float().mean().item()
    assert frac(got, attention_variant(q, k, v, 1.0, "reference")) < 0.01        # the same but for a summation order
    assert frac(got, attention_variant(q, k, v, 1.0, "unrounded")) > 0.2
    assert frac(got, attention_variant(q, k, v, 1.0, "both")) > 0.2


def test_a_model_without_layers_is_head_of_norm_of_embedding(tmp_path):
    # src/exec/dense_swiglu_model.rs:276-359; the reference's fixture is tests/support/model_families/qwen3.rs:26-36.
    from vosti_amd.config import Qwen3Config
    from vosti_amd.weights import write_random_model
    cfg = Qwen3Config(**dict(TINY["A"][0], num_hidden_layers=0, tie_word_embeddings=False))
    write_random_model(cfg, 4, tmp_path, dtype=torch.float32)
    m = plain.PlainQwen3(tmp_path, F32)
    ids = [3, 200, 3, 77]
    e = m.w["model.embed_tokens.weight"][torch.tensor(ids)]
    ref = plain.rms_norm(e, m.w["model.norm.weight"], m.eps, F32) @ m.w["lm_head.weight"].t()
    torch.testing.assert_close(m.logits(ids), ref)
    assert torch.equal(m.logits(ids)[0], m.logits(ids)[2])       # no layer mixes positions
