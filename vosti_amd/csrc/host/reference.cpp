// Plain references of the GPU kernels: straight loops on the host, one function per kernel.
//
// They compute what the kernels in csrc/*.hip compute, with the same formulas and, where an order of
// summation is part of a kernel's contract, in that order:
//   * projections: K in chunks of 512 from 0; within a chunk the products are added to a sum that starts
//     at zero, slab (64 bytes of a row) after slab, and inside a slab in the order in which mma_slab
//     feeds the matrix unit; the chunk sums are added to a zero total in chunk order (gemm.hip);
//   * attention: keys in tiles of 64 at absolute positions; a segment of four tiles takes its tiles in, ascending,
//     onto a running state (a reference maximum that moves when the tile's exceeds it by more than 2^8, the sums
//     so far scaled when it moves, the tile's products added); the segments are folded into the total in ascending
//     order (attention.hip).
// Storage is float everywhere; `bf16` != 0 rounds every value that the kernels store in the element
// type to bfloat16 (round to nearest even), which is where the reference engine rounds too
// (every formula cites its source in the kernel's own file).
//
// They are slow on purpose and share no code with the kernels.  Tests compare the kernels with them
// (tests/test_reference_gpu.py) and them with the plain Python implementation (tests/test_reference_cpu.py).
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

inline float round_bf16(float x) {
  uint32_t u;
  std::memcpy(&u, &x, 4);
  if ((u & 0x7f800000u) == 0x7f800000u) {          // inf or nan: keep the class
    if (u & 0x007fffffu) u |= 0x00400000u;
    u &= 0xffff0000u;
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);               // nearest, ties to even
    u &= 0xffff0000u;
  }
  float y;
  std::memcpy(&y, &u, 4);
  return y;
}

inline float store(float x, int bf16) { return bf16 ? round_bf16(x) : x; }

constexpr int KC = 512;          // elements of a chunk
constexpr int TILE_KEYS = 64;
constexpr int SEG_TILES = 4;

// 2^x as the fold and the probabilities use it.
inline float exp2_ref(float x) { return std::exp2(x); }

struct Partial {                 // (m, l, acc[d]) of a segment or a row
  float m = -INFINITY, l = 0.f;
  std::vector<float> acc;
  explicit Partial(int d) : acc(d, 0.f) {}
};

// state <- fold of a non-empty segment: M' = max(M, m); X' = fma(x, 2^(m - M'), X * 2^(M - M')).
void fold(Partial& S, const Partial& p) {
  if (!(p.m > -INFINITY)) return;
  const float Mn = std::fmax(S.m, p.m);
  const float ca = exp2_ref(S.m - Mn), cb = exp2_ref(p.m - Mn);
  for (size_t i = 0; i < S.acc.size(); ++i) S.acc[i] = std::fma(p.acc[i], cb, S.acc[i] * ca);
  S.l = std::fma(p.l, cb, S.l * ca);
  S.m = Mn;
}

}  // namespace

extern "C" {

float vh_ref_round_bf16(float x) { return round_bf16(x); }

// out[t] = table[ids[t]].
void vh_ref_embedding(float* out, const float* table, const int32_t* ids, int T, int H) {
  for (int t = 0; t < T; ++t) std::memcpy(out + (int64_t)t * H, table + (int64_t)ids[t] * H, sizeof(float) * H);
}

// y = (x * rsqrt(mean(x^2) + eps)) * w per row.
void vh_ref_rmsnorm(float* out, const float* x, const float* w, int rows, int H, float eps, int bf16) {
  for (int r = 0; r < rows; ++r) {
    const float* xr = x + (int64_t)r * H;
    float ss = 0.f;
    for (int i = 0; i < H; ++i) ss = ss + xr[i] * xr[i];
    const float rr = 1.0f / std::sqrt(ss / (float)H + eps);
    for (int i = 0; i < H; ++i) out[(int64_t)r * H + i] = store((xr[i] * rr) * w[i], bf16);
  }
}

// h = x + residual in float; residual <- h rounded; out = norm of the unrounded h.
void vh_ref_add_rmsnorm(float* out, float* residual, const float* x, const float* w, int rows, int H, float eps,
                        int bf16) {
  std::vector<float> h(H);
  for (int r = 0; r < rows; ++r) {
    float ss = 0.f;
    for (int i = 0; i < H; ++i) {
      h[i] = x[(int64_t)r * H + i] + residual[(int64_t)r * H + i];
      ss = ss + h[i] * h[i];
    }
    const float rr = 1.0f / std::sqrt(ss / (float)H + eps);
    for (int i = 0; i < H; ++i) {
      residual[(int64_t)r * H + i] = store(h[i], bf16);
      out[(int64_t)r * H + i] = store((h[i] * rr) * w[i], bf16);
    }
  }
}

// out[M, N] = act[M, K] w[N, K]^T in the kernels' order.  A slab is 64 bytes of a row: 16 floats, or 32
// bfloat16.  In a float slab the matrix unit is fed four times, with the elements {j, 4 + j, 8 + j, 12 + j}
// for j = 0..3, and adds the four products of a feed one after the other, each product fused into the
// sum; in a bfloat16 slab it is fed once with all 32 products, which are exact in float and are added
// here in ascending order (the unit's own order inside one feed is not documented).
void vh_ref_gemm(float* out, const float* act, const float* w, int M, int N, int K, int bf16) {
  const int slab = bf16 ? 32 : 16;
  for (int m = 0; m < M; ++m) {
    for (int n = 0; n < N; ++n) {
      const float* a = act + (int64_t)m * K;
      const float* b = w + (int64_t)n * K;
      float total = 0.f;
      for (int c0 = 0; c0 < K; c0 += KC) {
        const int c1 = c0 + KC < K ? c0 + KC : K;
        float acc = 0.f;
        for (int s0 = c0; s0 < c1; s0 += slab) {
          if (bf16) {
            for (int i = s0; i < s0 + slab && i < c1; ++i) acc = acc + b[i] * a[i];
          } else {
            for (int j = 0; j < 4; ++j)
              for (int g = 0; g < 4; ++g) {
                const int i = s0 + 4 * g + j;
                if (i < c1) acc = std::fma(b[i], a[i], acc);
              }
          }
        }
        total = total + acc;
      }
      out[(int64_t)m * N + n] = store(total, bf16);
    }
  }
}

// out[t, i] = silu(g) * u with g = gu[t, i], u = gu[t, I + i].
void vh_ref_swiglu(float* out, const float* gu, int T, int I, int bf16) {
  for (int t = 0; t < T; ++t)
    for (int i = 0; i < I; ++i) {
      const float g = gu[(int64_t)t * 2 * I + i], u = gu[(int64_t)t * 2 * I + I + i];
      out[(int64_t)t * I + i] = store((g * (1.0f / (1.0f + std::exp(-g)))) * u, bf16);
    }
}

// Head norm (weights may be null: no norm), half rotation of the first 2 * rot_half elements of a head
// (tables may be null: no rotation), store of k and v at their slots (slot -1: nothing; nkv 0: no store).
// qkv [T, (nq + 2 nkv) d]; q_out [T, nq, d]; kc [pages, nkv, P, d]; vc [pages, nkv, d, P].
void vh_ref_qkv_post(float* q_out, float* kc, float* vc, const float* qkv, const float* q_w, const float* k_w,
                     const float* cos_t, const float* sin_t, int rot_half, const int32_t* positions,
                     const int32_t* slots, int T, int nq, int nkv, int d, int P, float eps, int bf16) {
  const int width = (nq + 2 * nkv) * d;
  std::vector<float> y(d);
  for (int t = 0; t < T; ++t) {
    for (int h = 0; h < nq + 2 * nkv; ++h) {
      const float* x = qkv + (int64_t)t * width + (int64_t)h * d;
      const int kind = h < nq ? 0 : (h < nq + nkv ? 1 : 2);
      const float* w = kind == 0 ? q_w : (kind == 1 ? k_w : nullptr);
      for (int i = 0; i < d; ++i) y[i] = x[i];
      if (w != nullptr) {
        float ss = 0.f;
        for (int i = 0; i < d; ++i) ss = ss + x[i] * x[i];
        const float rr = 1.0f / std::sqrt(ss / (float)d + eps);
        for (int i = 0; i < d; ++i) y[i] = store((x[i] * rr) * w[i], bf16);
      }
      if (cos_t != nullptr && kind != 2) {
        const float* c = cos_t + (int64_t)positions[t] * rot_half;
        const float* s = sin_t + (int64_t)positions[t] * rot_half;
        for (int i = 0; i < rot_half; ++i) {
          const float x1 = y[i], x2 = y[i + rot_half];
          y[i] = store(x1 * c[i] - x2 * s[i], bf16);
          y[i + rot_half] = store(x2 * c[i] + x1 * s[i], bf16);
        }
      }
      if (kind == 0) {
        for (int i = 0; i < d; ++i) q_out[((int64_t)t * nq + h) * d + i] = y[i];
      } else if (slots != nullptr && slots[t] >= 0) {
        const int page = slots[t] / P, off = slots[t] % P;
        if (kind == 1) {
          const int kh = h - nq;
          for (int i = 0; i < d; ++i) kc[(((int64_t)page * nkv + kh) * P + off) * d + i] = y[i];
        } else {
          const int kh = h - nq - nkv;
          for (int i = 0; i < d; ++i) vc[(((int64_t)page * nkv + kh) * d + i) * P + off] = y[i];
        }
      }
    }
  }
}

// Causal grouped-query attention over the paged cache for every row of every sequence.  Row r of a
// sequence with q_len rows and k_len keys stands at position k_len - q_len + r and sees the keys
// max(0, p - window + 1) .. p (all from 0 without a window).  Tiles, segments and total as in attention.hip.
void vh_ref_paged_attention(float* out, const float* q, const float* kc, const float* vc, const int32_t* block_table,
                            int bt_stride, const int32_t* cu_q, const int32_t* k_len, int S, int nq, int nkv, int d,
                            int P, int window, float scale, int bf16) {
  const float c = scale * 1.4426950408889634f;
  const int G = nq / nkv;
  std::vector<float> sc(TILE_KEYS), pr(TILE_KEYS);
  for (int s = 0; s < S; ++s) {
    const int q_begin = cu_q[s], q_len = cu_q[s + 1] - q_begin, kl = k_len[s];
    const int32_t* bt = block_table + (int64_t)s * bt_stride;
    for (int r = 0; r < q_len; ++r) {
      const int pos = kl - q_len + r;
      const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
      for (int h = 0; h < nq; ++h) {
        const int kvh = h / G;
        const float* qr = q + ((int64_t)(q_begin + r) * nq + h) * d;
        Partial total(d);
        if (pos >= 0) {
          for (int seg = lo / (TILE_KEYS * SEG_TILES); seg <= pos / (TILE_KEYS * SEG_TILES); ++seg) {
            Partial sp(d);
            for (int t = seg * SEG_TILES; t < seg * SEG_TILES + SEG_TILES; ++t) {
              const int kb = t * TILE_KEYS;
              if (kb > pos || kb + TILE_KEYS <= lo) continue;
              float mx = -INFINITY;
              for (int j = 0; j < TILE_KEYS; ++j) {
                const int key = kb + j;
                if (key < lo || key > pos) continue;
                const float* kr = kc + (((int64_t)bt[key / P] * nkv + kvh) * P + key % P) * d;
                // The dot product over the head in the order of the projections' slabs.
                float acc = 0.f;
                if (bf16) {
                  for (int i = 0; i < d; ++i) acc = acc + kr[i] * qr[i];
                } else {
                  for (int s0 = 0; s0 < d; s0 += 16)
                    for (int jj = 0; jj < 4; ++jj)
                      for (int g = 0; g < 4; ++g) acc = std::fma(kr[s0 + 4 * g + jj], qr[s0 + 4 * g + jj], acc);
                }
                sc[j] = acc;
                mx = std::fmax(mx, acc);
              }
              if (!(mx > -INFINITY)) continue;         // the row sees no key of the tile: its state stands
              // The tile onto the segment's state: the new maximum, the sums so far under it, the tile's own added.
              // The reference point moves only when the state is empty or the maximum grows by more than 2^8.
              const float mt = mx * c;
              const float Mn = (!(sp.m > -INFINITY) || mt > sp.m + 8.0f) ? mt : sp.m;
              const float ca = exp2_ref(sp.m - Mn);      // 1 where the maximum stands, 0 while the state is empty
              float l = 0.f;
              for (int j = 0; j < TILE_KEYS; ++j) {
                const int key = kb + j;
                pr[j] = (key < lo || key > pos) ? 0.f : exp2_ref(std::fma(sc[j], c, -Mn));
                l = l + pr[j];
              }
              sp.l = std::fma(sp.l, ca, l);
              sp.m = Mn;
              for (int i = 0; i < d; ++i) {
                float a = sp.acc[i] * ca;
                for (int j = 0; j < TILE_KEYS; ++j) {
                  const int key = kb + j;
                  if (key < lo || key > pos) continue;
                  const float v = vc[(((int64_t)bt[key / P] * nkv + kvh) * d + i) * P + key % P];
                  a = a + v * store(pr[j], bf16);
                }
                sp.acc[i] = a;
              }
            }
            fold(total, sp);
          }
        }
        const float inv = total.l > 0.f ? 1.0f / total.l : 0.f;
        for (int i = 0; i < d; ++i) out[((int64_t)(q_begin + r) * nq + h) * d + i] = store(total.acc[i] * inv, bf16);
      }
    }
  }
}

// First index of the maximum; a NaN counts as the maximum; an empty row gives 0.
int vh_ref_argmax(const float* row, int V) {
  int best = 0x7fffffff;
  float bv = -INFINITY;
  for (int i = 0; i < V; ++i) {
    const float v = row[i];
    const bool vn = v != v, bn = bv != bv;
    const bool better = vn ? (!bn || i < best) : (bn ? false : (v > bv || (v == bv && i < best)));
    if (better) {
      bv = v;
      best = i;
    }
  }
  return best == 0x7fffffff ? 0 : best;
}

// Temperature sampling by inverse CDF, in the sampler's order: the vocabulary in 1024 contiguous ranges
// of ceil(V / 1024), each summed in ascending order, the range sums scanned in order, the target
// u * total looked up first by range, then inside the range.  temp <= 0, a NaN or +inf maximum: argmax.
int vh_ref_sample(const float* row, int V, float temp, float u) {
  const int imax = vh_ref_argmax(row, V);
  const float vmax = row[imax];
  if (!(temp > 0.f) || vmax != vmax || vmax == INFINITY) return imax;
  const int R = 1024, C = (V + R - 1) / R;
  const float zmax = vmax / temp;
  std::vector<float> sum(R, 0.f), pre(R + 1, 0.f);
  for (int t = 0; t < R; ++t) {
    const int lo = t * C < V ? t * C : V, hi = lo + C < V ? lo + C : V;
    float sm = 0.f;
    for (int i = lo; i < hi; ++i) sm = sm + std::exp(row[i] / temp - zmax);
    sum[t] = sm;
  }
  float run = 0.f;
  for (int t = 0; t < R; ++t) {
    pre[t] = run;
    run = run + sum[t];
  }
  pre[R] = run;
  const float target = u * run;
  int own = -1, last = 0;
  for (int t = 0; t < R; ++t)
    if (sum[t] > 0.f) {
      last = t;
      if (own < 0 && target < pre[t + 1]) own = t;
    }
  if (own < 0) own = last;
  const int lo = own * C < V ? own * C : V, hi = lo + C < V ? lo + C : V;
  float acc = pre[own];
  int pick = -1, last_pos = lo;
  for (int i = lo; i < hi; ++i) {
    const float e = std::exp(row[i] / temp - zmax);
    acc = acc + e;
    if (e > 0.f) last_pos = i;
    if (pick < 0 && target < acc) pick = i;
  }
  return pick >= 0 ? pick : last_pos;
}

}  // extern "C"
