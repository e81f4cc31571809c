"""The sizes that the measurements run at: the vocabulary of 151,936 entries through the head projection, the
sampler and the embedding; decode steps of 48 and 64 rows through both step functions; decoded tokens over
33,000 keys.  The other kernel tests use sizes of their own."""
import random

import pytest
import torch

import plain_qwen3 as plain
from test_kernels_gpu import kern, rand, run_attention, tol

pytestmark = pytest.mark.gpu

VOCAB = 151936


def device_normal(shape, dtype, seed, scale):
    """Normal values drawn on the GPU (a matrix of 151,936 rows takes the CPU's generator too long)."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("K", [4096, 1024])
def test_head_projection_at_the_vocabulary(dtype, K):
    """The vocabulary projection of the measured shapes (151,936 x 4,096, and x 1,024 of the small tied
    shapes) at 1, 8 and 64 rows: against a product in 64-bit on the CPU (the reference's tolerances for its
    own products, kernels/benchmarks/matmul.py:54, are wider than these), every row of a batch equal to
    the row alone bit for bit (:55-58), and with a workspace the same bits."""
    k = kern(dtype)
    w = device_normal((VOCAB, K), dtype, 1, K ** -0.5)
    a = device_normal((64, K), dtype, 2, 1.0)
    w64, a64 = w.cpu(), a.cpu().double()
    ref = torch.empty(64, VOCAB, dtype=torch.float32)
    for lo in range(0, VOCAB, 16384):            # in pieces: the whole matrix in 64-bit would be 5 GB
        ref[:, lo:lo + 16384] = (a64 @ w64[lo:lo + 16384].double().t()).float()
    del w64
    ws = torch.empty(max(k.gemm_workspace_floats(64, VOCAB, K, force=True), 1), device="cuda")
    full = None
    for M in (64, 8, 1):
        got = k.gemm(a[:M], w)
        torch.testing.assert_close(got.float().cpu(), ref[:M].to(dtype).float(), **tol(dtype))
        if full is None:
            full = got
        assert torch.equal(got, full[:M]), f"{M} rows alone and as the first rows of 64"
        assert torch.equal(k.gemm(a[:M], w, workspace=ws), got), f"{M} rows with a workspace"
        # The last vocabulary entries (the last, partly filled weight tiles) are not left out.
        assert got[:, -40:].float().abs().sum() > 0
    for r in (0, 37, 63):
        assert torch.equal(k.gemm(a[r:r + 1], w)[0], full[r])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_sampler_at_the_vocabulary(dtype):
    """Greedy: the largest logit in the last entries, in the first, in the middle, and twice (the first one wins).
    At a temperature: the drawn token's interval of the 64-bit CDF holds the uniform number."""
    k = kern(dtype)
    rows = 64
    logits = rand((rows, VOCAB), dtype, 3, 2.0)
    where = [VOCAB - 1, 0, VOCAB // 2, VOCAB - 7, VOCAB - 300, 148 * 1024 - 1, 148 * 1024, 77777]
    for r, v in enumerate(where):
        logits[r, v] = 30.0
    logits[8, 1000] = logits[8, VOCAB - 2] = 31.0           # a tie: the lower index
    got = k.sample(logits.cuda()).cpu().tolist()
    assert got[:8] == where and got[8] == 1000
    want = torch.argmax(logits.float(), dim=1).tolist()
    assert got[:8] + got[9:] == want[:8] + want[9:]
    assert k.sample(logits[:8].cuda()).cpu().tolist() == got[:8] and k.sample(logits[7:8].cuda()).cpu().tolist() == got[7:8]
    plainer = rand((8, VOCAB), dtype, 4, 2.0)
    temps = torch.tensor([0.7, 1.3, 0.0, 0.7, 1.0, 0.2, 2.0, 1.0])
    u = torch.tensor([0.25, 0.9, 0.5, 0.25, 1 - 2 ** -24, 0.0, 0.999, 0.5])
    drawn = k.sample(plainer.cuda(), temps.cuda(), u.cuda()).cpu().tolist()
    for r in range(8):
        if temps[r] == 0:
            assert drawn[r] == int(torch.argmax(plainer[r].float()))
            continue
        cdf = torch.cumsum(torch.softmax(plainer[r].double() / temps[r].double(), dim=0), dim=0)
        lo = cdf[drawn[r] - 1] if drawn[r] > 0 else 0.0
        assert 0 <= drawn[r] < VOCAB and lo - 2e-4 <= u[r] <= cdf[drawn[r]] + 2e-4, (r, drawn[r])
    assert k.sample(plainer[3:4].cuda(), temps[3:4].cuda(), u[3:4].cuda()).item() == drawn[3]     # alone: the same token


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_embedding_at_the_vocabulary(dtype):
    k = kern(dtype)
    table = device_normal((VOCAB, 4096), dtype, 5, 1.0)
    ids = torch.tensor([0, VOCAB - 1, 65536, 131072, VOCAB - 1, 7], dtype=torch.int32)
    got = k.embedding(table, ids.cuda())
    assert torch.equal(got, table[ids.long().cuda()])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_decoded_tokens_over_33000_keys(dtype):
    """33,000 keys (129 segments of 256): a decoded token against the plain row, alone and beside seven
    shorter ones, with NaN in every unused page and tail; and a key that outweighs all others in the first
    tile, in the last full segment and at the very end."""
    k = kern(dtype)
    nq, nkv, d, P, L = 8, 2, 128, 64, 33000
    lens = [L, 31999, 2048, 257, 20000, 1, 4097, 32768]
    q_list = [rand((1, nq, d), dtype, 10 + i) for i in range(len(lens))]
    kk = [rand((n, nkv, d), dtype, 40 + i) for i, n in enumerate(lens)]
    vv = [rand((n, nkv, d), dtype, 70 + i) for i, n in enumerate(lens)]
    got = run_attention(k, q_list, kk, vv, P, dtype, poison=float("nan"))
    for i in (0, 1, 4, 7):
        ref = plain.attention(q_list[i], kk[i], vv[i], d ** -0.5, dtype)
        torch.testing.assert_close(got[i:i + 1].float(), ref, **tol(dtype))
    alone = run_attention(k, q_list[:1], kk[:1], vv[:1], P, dtype, seed=9)
    assert torch.equal(alone[0], got[0])
    for far in (5, 32767, L - 1):
        q2, k2 = q_list[0].clone() * 0.1, kk[0].clone() * 0.1
        q2[:, :, 0] = 40.0
        k2[far, :, 0] = 40.0
        out = run_attention(k, [q2], [k2], [vv[0]], P, dtype)
        torch.testing.assert_close(out[0].float(), vv[0][far].float().repeat_interleave(nq // nkv, dim=0), **tol(dtype))


@pytest.mark.parametrize("rows", [48, 64])
def test_wide_decode_steps_through_both_step_functions(tmp_path_factory, rows):
    """Two layers of the measured width with 48 and 64 requests decoding together, the steps replayed from
    recordings (the sizes of the measurement's batch of 64: projections of 33 to 64 rows, the sampler and the
    attention at that many rows).  Through the native engine and through the Python one the tokens are the
    same, and those of a request are the tokens it generates when it runs alone."""
    from vosti_amd.config import Qwen3Config
    from vosti_amd.engine import Engine, NativeEngine
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import write_random_model
    V = 4999
    d = tmp_path_factory.mktemp(f"wide{rows}")
    cfg = Qwen3Config(vocab_size=V, hidden_size=4096, intermediate_size=12288, num_hidden_layers=2, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, max_position_embeddings=1024, rms_norm_eps=1e-6, rope_theta=1e6,
                      tie_word_embeddings=False)
    write_random_model(cfg, 13, d)
    rng = random.Random(rows)
    ps = [[rng.randrange(V) for _ in range(rng.choice((3, 20, 64, 65, 130, 300)))] for _ in range(rows)]
    sp = [SamplingParams(max_tokens=9, temperature=0.8 if i % 5 == 2 else 0.0, seed=i, ignore_eos=True) for i in range(rows)]
    kw = dict(dtype="bfloat16", num_pages=rows * 6, page_size=64, max_num_seqs=rows, max_num_batched_tokens=8192, graphs=True)
    native = NativeEngine(d, **kw)
    got = native.generate(ps, sp)
    st = native.stats()["graph_stats"]
    assert st["replayed"] >= 6 and native.cache_check() == ""
    python = Engine(str(d), **kw)
    assert python.generate(ps, sp) == got
    assert python.runner.graph_stats == st
    # Alone, with nothing recorded and nothing beside it.
    single = NativeEngine(d, **dict(kw, num_pages=8, max_num_seqs=1, graphs=False))
    for i in list(range(0, rows, 5)) + [rows - 1]:
        assert single.generate([ps[i]], sp[i]) == [got[i]], f"request {i}"
