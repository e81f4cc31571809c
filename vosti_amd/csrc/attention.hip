// Causal grouped-query attention over the paged cache, for prompt portions and
// decoded tokens alike, with an optional sliding window.
//
// What is computed is the reference's kernel
// (kernels/triton_kernels/fattn_paged.py:126-277): row r of a sequence with
// q_len new tokens and k_len keys stands at position p = k_len - q_len + r and
// sees keys lo..p (lo = 0, or p - window + 1 with a window); q head h reads kv
// head h / (nq / nkv); scores are (q.k) * scale * log2(e); softmax in base 2 with
// fp32 statistics; probabilities are rounded to the element type before P.V; a
// tile in which a row sees no key leaves that row's state untouched; out =
// acc / l (0 if l == 0).
//
// Reduction order (a function of absolute key positions only, so that any cut
// of a sequence into steps, and any split of the keys over workgroups, gives
// the same bits):
//   keys are grouped in tiles of 64 (positions 64t .. 64t+63) and tiles in
//   segments of 4 (256 keys).  Within a segment the state (m, l, acc) starts
//   at (-inf, 0, 0) and is updated tile by tile, ascending, by online softmax.
//   Segment results are merged into the total, ascending:
//     M' = max(M, m); ACC' = ACC * 2^(M - M') + acc * 2^(m - M'); L' likewise.
//   A workgroup either walks all segments of its rows and merges in registers
//   (prompt portions), or takes one segment and leaves (m, l, acc) in a
//   scratch buffer that attn_combine merges with the same formula (decode).
//
// Cache layout: keys [pages, nkv, page, d]; values transposed [pages, nkv, d, page],
// so that both MFMA operands of both products are 16-byte loads from global
// memory: S^T = K Q^T and O^T = V^T P^T, which keeps a query row in one lane
// column from scores to output.
#include "common.h"
#include "mma.h"
#include "vec.h"

#define TILE_KEYS 64
#define SEG_TILES 4
#define KEY_SLABS (TILE_KEYS / VK_SLAB)   // key slabs per tile: 2 (bfloat16) or 4 (float)
#define S_PER_LANE 16                     // scores per lane per tile

struct AttnArgs {
  const elem_t* q;        // [T, nq, d]
  elem_t* out;            // [T, nq, d]
  const elem_t* kc;       // [pages, nkv, P, d]
  const elem_t* vc;       // [pages, nkv, d, P]
  const int32_t* block_table;  // [S, bt_stride]
  const int32_t* cu_q;    // [S + 1]
  const int32_t* k_len;   // [S]
  const int32_t* items;   // [n_items, 2]: (sequence, first row of the item within the step's rows of it)
  float* part_ml;         // split: [T * nq * nseg, 2]
  float* part_acc;        // split: [T * nq * nseg, d]
  int bt_stride, nq, nkv, d, P, window, nseg;
  float scale_log2;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// MODE 0: the 16 rows of a wave are 16 consecutive tokens of one q head.
// MODE 1: the 16 rows are up to 16 q heads of one kv head, for one token.
template <int DPAD, int MODE, bool SPLIT>
__global__ __launch_bounds__(64) void attn_kernel(AttnArgs a) {
  constexpr int NDT = DPAD / 16;          // output d tiles
  constexpr int NQS = DPAD / VK_SLAB;     // slabs along d
  const int lane = threadIdx.x, r16 = lane & 15, g = lane >> 4;
  const int seq = a.items[2 * blockIdx.x], q_off = a.items[2 * blockIdx.x + 1];
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  const int k_len = a.k_len[seq];
  const int G = a.nq / a.nkv;
  const int d = a.d, P = a.P;

  int tok, head, kvh, pos, nvalid;
  if (MODE == 0) {
    head = blockIdx.y;
    kvh = head / G;
    nvalid = min(16, q_len - q_off);
    tok = q_begin + q_off + r16;
    pos = k_len - q_len + q_off + r16;
  } else {
    const int HT = (G + 15) >> 4;
    kvh = blockIdx.y / HT;
    const int ht = blockIdx.y - kvh * HT;
    nvalid = min(16, G - ht * 16);
    head = kvh * G + ht * 16 + r16;
    tok = q_begin + q_off;
    pos = k_len - q_len + q_off;
  }
  const bool row_ok = r16 < nvalid;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  // Key range that any row of this wave sees.
  const int pos0 = k_len - q_len + q_off;
  const int wave_hi = MODE == 0 ? pos0 + nvalid - 1 : pos0;
  const int wave_lo = a.window > 0 ? max(0, pos0 - a.window + 1) : 0;
  const int tile_lo = wave_lo / TILE_KEYS, tile_hi = wave_hi / TILE_KEYS;
  int seg_begin = tile_lo / SEG_TILES, seg_end = tile_hi / SEG_TILES + 1;
  if (SPLIT) {
    const int seg = blockIdx.z;
    if (seg < seg_begin || seg >= seg_end) return;
    seg_begin = seg;
    seg_end = seg + 1;
  }

  const int32_t* bt = a.block_table + (int64_t)seq * a.bt_stride;
  const int64_t page_elems = (int64_t)P * d;       // elements of one (page, kv head)
  const elem_t* kbase = a.kc + (int64_t)kvh * page_elems;
  const elem_t* vbase = a.vc + (int64_t)kvh * page_elems;
  const int64_t page_stride = (int64_t)a.nkv * page_elems;

  // Query fragments: second MFMA operand, lane (row r16, column group g).
  frag_t qf[NQS];
  {
    const elem_t* qrow = a.q + ((int64_t)tok * a.nq + head) * d;
#pragma unroll
    for (int s = 0; s < NQS; ++s) {
      const int c = s * VK_SLAB + g * VK_VEC;
      qf[s] = load_frag(qrow + (row_ok ? c : 0), row_ok && c < d);
    }
  }

  float M_tot = -INFINITY, L_tot = 0.f;
  f32x4 ACC[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) ACC[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int seg = seg_begin; seg < seg_end; ++seg) {
    float m_run = -INFINITY, l_run = 0.f;
    f32x4 acc[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int t_begin = max(tile_lo, seg * SEG_TILES), t_end = min(tile_hi, seg * SEG_TILES + SEG_TILES - 1);
    for (int t = t_begin; t <= t_end; ++t) {
      const int kb = t * TILE_KEYS;
      // ---- scores S^T[key, row] = K Q^T ----
      float sc[S_PER_LANE];
#pragma unroll
      for (int ks = 0; ks < KEY_SLABS; ++ks) {
#ifdef VK_BF16
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          // MFMA row m of this sub-tile is key  slab + 8*(m/4) + 4*u + m%4, so that
          // lane group g ends up with the 8 consecutive keys slab + 8g .. 8g+7.
          const int key = kb + ks * VK_SLAB + 8 * (r16 >> 2) + 4 * u + (r16 & 3);
#else
        {
          const int u = 0;
          const int key = kb + ks * VK_SLAB + r16;
#endif
          const bool kok = key < k_len;
          const int kk = kok ? key : 0;
          const int page = bt[kk / P];
          const elem_t* krow = kbase + page * page_stride + (int64_t)(kk % P) * d;
          f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < NQS; ++s) {
            if (s * VK_SLAB < d) {
              const int c = s * VK_SLAB + g * VK_VEC;
              const frag_t kf = load_frag(krow + c, kok && c < d);
              s4 = mma_slab(kf, qf[s], s4);
            }
          }
          sc[ks * VK_VEC + 4 * u + 0] = s4.x;
          sc[ks * VK_VEC + 4 * u + 1] = s4.y;
          sc[ks * VK_VEC + 4 * u + 2] = s4.z;
          sc[ks * VK_VEC + 4 * u + 3] = s4.w;
        }
      }
      // ---- mask, running max ----
      bool vis[S_PER_LANE];
      float tmax = -INFINITY;
      int any = 0;
#pragma unroll
      for (int i = 0; i < S_PER_LANE; ++i) {
        const int key = kb + (i / VK_VEC) * VK_SLAB + g * VK_VEC + (i % VK_VEC);
        vis[i] = row_ok && key >= lo && key <= pos;
        sc[i] = sc[i] * a.scale_log2;
        tmax = fmaxf(tmax, vis[i] ? sc[i] : -INFINITY);
        any |= vis[i] ? 1 : 0;
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, VK_WAVE));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, VK_WAVE));
      any |= __shfl_xor(any, 16, VK_WAVE);
      any |= __shfl_xor(any, 32, VK_WAVE);
      const float m_new = any ? fmaxf(m_run, tmax) : m_run;
      const float alpha = any ? fast_exp2(m_run - m_new) : 1.0f;
      float psum = 0.f;
      float pr[S_PER_LANE];
#pragma unroll
      for (int i = 0; i < S_PER_LANE; ++i) {
        pr[i] = vis[i] ? fast_exp2(sc[i] - m_new) : 0.f;
        psum = psum + pr[i];
      }
      psum = psum + __shfl_xor(psum, 16, VK_WAVE);
      psum = psum + __shfl_xor(psum, 32, VK_WAVE);
      l_run = any ? l_run * alpha + psum : l_run;
      m_run = m_new;
      // ---- P fragments (second operand of O^T = V^T P^T), rounded to the element type ----
      frag_t pf[KEY_SLABS];
#pragma unroll
      for (int ks = 0; ks < KEY_SLABS; ++ks) {
#ifdef VK_BF16
#pragma unroll
        for (int j = 0; j < 8; ++j) pf[ks][j] = (__bf16)pr[ks * 8 + j];
#else
        pf[ks] = f32x4{pr[ks * 4 + 0], pr[ks * 4 + 1], pr[ks * 4 + 2], pr[ks * 4 + 3]};
#endif
      }
      // ---- acc = acc * alpha + V^T P^T ----
      // Keys outside [wave_lo, k_len) may lie in pages this sequence does not own
      // (never written, or given back once the window passed them): their values
      // are replaced by zero so that stale NaN or Inf cannot reach the sum.
      const bool edge = kb + TILE_KEYS > k_len || kb < wave_lo;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        if (dt * 16 < d) {
          acc[dt].x = acc[dt].x * alpha; acc[dt].y = acc[dt].y * alpha;
          acc[dt].z = acc[dt].z * alpha; acc[dt].w = acc[dt].w * alpha;
#pragma unroll
          for (int ks = 0; ks < KEY_SLABS; ++ks) {
            const int k0 = kb + ks * VK_SLAB + g * VK_VEC;
            const bool vok = k0 < k_len;
            const int kk = vok ? k0 : 0;
            const int page = bt[kk / P];
            const elem_t* vrow = vbase + page * page_stride + (int64_t)(dt * 16 + r16) * P + (kk % P);
            frag_t vf = load_frag(vrow, vok);
            if (edge) {
#pragma unroll
              for (int j = 0; j < VK_VEC; ++j)
                if (k0 + j >= k_len || k0 + j < wave_lo) vf[j] = (elem_t)0.f;
            }
            acc[dt] = mma_slab(vf, pf[ks], acc[dt]);
          }
        }
      }
    }
    // ---- leave the segment ----
    if (SPLIT) {
      if (row_ok) {
        const int64_t prow = ((int64_t)tok * a.nq + head) * a.nseg + seg;
        if (g == 0) {
          a.part_ml[2 * prow] = m_run;
          a.part_ml[2 * prow + 1] = l_run;
        }
        if (m_run > -INFINITY) {
#pragma unroll
          for (int dt = 0; dt < NDT; ++dt)
            if (dt * 16 < d) *reinterpret_cast<f32x4*>(a.part_acc + prow * d + dt * 16 + 4 * g) = acc[dt];
        }
      }
    } else if (m_run > -INFINITY) {
      const float Mn = fmaxf(M_tot, m_run);
      const float ca = fast_exp2(M_tot - Mn), cb = fast_exp2(m_run - Mn);
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        ACC[dt].x = ACC[dt].x * ca + acc[dt].x * cb; ACC[dt].y = ACC[dt].y * ca + acc[dt].y * cb;
        ACC[dt].z = ACC[dt].z * ca + acc[dt].z * cb; ACC[dt].w = ACC[dt].w * ca + acc[dt].w * cb;
      }
      L_tot = L_tot * ca + l_run * cb;
      M_tot = Mn;
    }
  }
  if (!SPLIT && row_ok) {
    const float inv = L_tot > 0.f ? 1.0f / L_tot : 0.f;
    elem_t* orow = a.out + ((int64_t)tok * a.nq + head) * d;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      if (dt * 16 < d) {
        const float o[4] = {ACC[dt].x * inv, ACC[dt].y * inv, ACC[dt].z * inv, ACC[dt].w * inv};
        elem_t* p = orow + dt * 16 + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; ++i) p[i] = from_f32<elem_t>(o[i]);
      }
    }
  }
}

// Merges the segment results of one (token, head) in ascending segment order.
// One wave per row; lane j owns output columns j, j+64, ...
__global__ __launch_bounds__(64) void attn_combine_kernel(AttnArgs a) {
  const int seq = a.items[2 * blockIdx.x], q_off = a.items[2 * blockIdx.x + 1];
  const int head = blockIdx.y;
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  const int k_len = a.k_len[seq];
  const int tok = q_begin + q_off;
  const int pos = k_len - q_len + q_off;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int seg_begin = lo / (TILE_KEYS * SEG_TILES), seg_end = pos / (TILE_KEYS * SEG_TILES) + 1;
  const int d = a.d;
  float M_tot = -INFINITY, L_tot = 0.f;
  float ACC[4] = {0.f, 0.f, 0.f, 0.f};   // d <= 256
  const int64_t row0 = ((int64_t)tok * a.nq + head) * a.nseg;
  for (int seg = seg_begin; seg < seg_end; ++seg) {
    const float m_run = a.part_ml[2 * (row0 + seg)], l_run = a.part_ml[2 * (row0 + seg) + 1];
    if (m_run > -INFINITY) {
      const float Mn = fmaxf(M_tot, m_run);
      const float ca = fast_exp2(M_tot - Mn), cb = fast_exp2(m_run - Mn);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = threadIdx.x + 64 * i;
        if (c < d) ACC[i] = ACC[i] * ca + a.part_acc[(row0 + seg) * d + c] * cb;
      }
      L_tot = L_tot * ca + l_run * cb;
      M_tot = Mn;
    }
  }
  const float inv = L_tot > 0.f ? 1.0f / L_tot : 0.f;
  elem_t* orow = a.out + ((int64_t)tok * a.nq + head) * d;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = threadIdx.x + 64 * i;
    if (c < d) orow[c] = from_f32<elem_t>(ACC[i] * inv);
  }
}

template <int MODE, bool SPLIT>
static void launch_attn(int dpad, dim3 grid, const AttnArgs& a, hipStream_t st) {
  if (dpad <= 64) attn_kernel<64, MODE, SPLIT><<<grid, 64, 0, st>>>(a);
  else if (dpad <= 128) attn_kernel<128, MODE, SPLIT><<<grid, 64, 0, st>>>(a);
  else attn_kernel<256, MODE, SPLIT><<<grid, 64, 0, st>>>(a);
}

extern "C" {

// Number of floats of scratch a split launch needs for `tokens` rows.
int64_t vk_attn_scratch_floats(int tokens, int nq, int d, int nseg) {
  const int64_t rows = (int64_t)tokens * nq * nseg;
  return ((rows * 2 + 3) & ~(int64_t)3) + rows * d;
}

int vk_attn_segment_keys(void) { return TILE_KEYS * SEG_TILES; }

// items: n_items pairs (sequence, first row).  mode 0: each item is up to 16
// consecutive rows of the sequence's q_len new tokens, fused over segments.
// mode 1: each item is one token; with split != 0 the keys are split by segment
// over nseg workgroups (scratch must hold vk_attn_scratch_floats(T, ...)) and
// merged by a second kernel.  The result is the same in every mode.
int vk_paged_attention(elem_t* out, const elem_t* q, const elem_t* kc, const elem_t* vc,
                       const int32_t* block_table, int bt_stride, const int32_t* cu_q, const int32_t* k_len,
                       const int32_t* items, int n_items, int mode, int split, int nseg, float* scratch,
                       int total_tokens, int nq, int nkv, int d, int P, int window, float scale,
                       hipStream_t st) {
  VK_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "attention: %d q heads are not a multiple of %d kv heads", nq, nkv);
  VK_REQUIRE(d >= 16 && d <= 256 && d % 16 == 0, "attention: head size %d must be a multiple of 16 in 16..256", d);
  VK_REQUIRE(P >= 8 && (P & (P - 1)) == 0, "attention: page size %d must be a power of two >= 8", P);
  VK_REQUIRE(window >= 0, "attention: window %d must not be negative", window);
  VK_REQUIRE(mode == 0 || mode == 1, "attention: unknown mode %d", mode);
  VK_REQUIRE(!(split && mode == 0), "attention: split is for single-token items only");
  VK_REQUIRE(nq <= 65535, "attention: too many heads");
  if (n_items <= 0) return 0;
  AttnArgs a;
  a.q = q; a.out = out; a.kc = kc; a.vc = vc; a.block_table = block_table; a.cu_q = cu_q; a.k_len = k_len;
  a.items = items; a.bt_stride = bt_stride; a.nq = nq; a.nkv = nkv; a.d = d; a.P = P; a.window = window;
  a.nseg = nseg; a.scale_log2 = scale * 1.4426950408889634f;
  a.part_ml = nullptr; a.part_acc = nullptr;
  const int G = nq / nkv;
  if (mode == 0) {
    launch_attn<0, false>(d, dim3(n_items, nq, 1), a, st);
  } else if (!split) {
    launch_attn<1, false>(d, dim3(n_items, nkv * ((G + 15) / 16), 1), a, st);
  } else {
    VK_REQUIRE(nseg > 0 && nseg <= 65535 && scratch != nullptr, "attention: split needs nseg in 1..65535 and scratch");
    a.part_ml = scratch;
    a.part_acc = scratch + (((int64_t)total_tokens * nq * nseg * 2 + 3) & ~(int64_t)3);
    launch_attn<1, true>(d, dim3(n_items, nkv * ((G + 15) / 16), nseg), a, st);
    if (vk_check_launch("attention")) return 1;
    attn_combine_kernel<<<dim3(n_items, nq), 64, 0, st>>>(a);
  }
  return vk_check_launch("attention");
}

}  // extern "C"
