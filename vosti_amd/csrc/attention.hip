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
// Reduction order.  It is a function of absolute key positions only, so that
// any cut of a sequence into steps, and any split of the keys over waves and
// workgroups, gives the same bits:
//   tile     64 keys, positions 64t .. 64t+63.
//   segment  4 tiles (256 keys).  A row's state (M, L, ACC) of a segment starts empty (M = -inf) and takes
//            in the segment's tiles in ascending order, each as the reference's kernel takes in a block of
//            keys (fattn_paged.py:198-262): with c = scale * log2(e) and m = (max of the tile's visible raw
//            scores) * c,
//              M' = m if the state is empty or m > M + 8, else M (the reference point moves only when the
//              maximum grows by more than 2^8: a probability is then at most 2^8, and the sums so far are
//              scaled in few tiles instead of in most); a = 2^(M - M');
//              p = 2^(fma(raw, c, -M')) (0 for a key the row does not see);
//              L' = fma(L, a, sum p); ACC' = ACC * a + P V, the product accumulated onto ACC * a by the
//            matrix unit, key slab after key slab.  A tile in which the row sees no key changes nothing.
//   total    the non-empty segments are folded, ascending, into a state that starts empty:
//              M' = max(M, m); ACC' = fma(acc, 2^(m - M'), ACC * 2^(M - M')); L' likewise.
// Kernels, all with the same sequence of fp32 operations per row:
//   attn_prefill_lds   prompt rows, head sizes 64/128/256 and pages of a tile or more: key and value
//                      tiles pass through LDS once per workgroup; segments and total in registers.
//   attn_prefill       prompt rows of every shape: fragments straight from global memory.
//   attn_decode_seg    decoded tokens: a wave walks the tiles of a segment with the next tile's
//                      fragments in flight; the segment's (M, L, ACC) goes to a scratch buffer ...
//   attn_combine       ... which this one folds.
//   attn_decode_pair   the same with two waves a segment, for steps with few segments.
//   attn_decode_plain  the same with a tile's fragments asked for when they are needed: for head and
//                      element sizes whose fragments of two tiles do not fit a wave's registers.
//
// Cache layout: keys [pages, nkv, page, d]; values transposed [pages, nkv, d, page],
// so that both MFMA operands of both products are 16-byte loads from global
// memory: S^T = K Q^T and O^T = V^T P^T, which keeps a query row in one lane
// column from scores to output.
#include <type_traits>

#include "common.h"
#include "mma.h"
#include "vec.h"

#define TILE_KEYS 64
#define SEG_TILES 4
#define KEY_SLABS (TILE_KEYS / VK_SLAB)   // key slabs per tile: 2 (bfloat16) or 4 (float)
#define S_PER_LANE 16                     // scores per lane per tile
#define ITEM_ROWS 128                     // rows of a prompt item
#define MAX_STEP 8.0f                     // a row's reference maximum moves when the tile's exceeds it by more than this (log2)

struct AttnArgs {
  const elem_t* q;        // [T, nq, d]
  elem_t* out;            // [T, nq, d]
  const elem_t* kc;       // [pages, nkv, P, d]
  const elem_t* vc;       // [pages, nkv, d, P]
  const int32_t* block_table;  // [S, bt_stride]
  const int32_t* cu_q;    // [S + 1]
  const int32_t* k_len;   // [S]
  const int32_t* items;   // [n_items, 2]: (sequence, first row of the item within the step's rows of it)
  float* part_ml;         // decode: [n_items * nq * nseg, 2], indexed by the item, not by the token
  float* part_acc;        // decode: [n_items * nq * nseg, d]
  int bt_stride, nq, nkv, d, P, window, nseg;
  float scale_log2;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// What a wave needs to know about its 16 rows and its sequence's pages.
struct RowCtx {
  const int32_t* bt;
  const elem_t* kbase;     // + kv head offset
  const elem_t* vbase;
  int64_t page_stride;
  int k_len, d, P, lp, r16, g;   // lp = log2(P)
  int lo, pos;             // this lane's row sees keys lo..pos
  int wave_lo;             // smallest key any row of the wave sees
  bool row_ok;
  float scale_log2;
};

// Scores of one tile onto the running state (M, L) of this lane's row in its segment: the new reference
// maximum (see the top of this file), the factor `ca` that the row's sums so far have to be scaled by (ACC is the
// caller's), L, and the tile's probabilities relative to the new maximum, rounded to the element type, as MFMA
// operands.  The row sees keys
// lo..pos.  A probability is 2^(score * scale_log2 - M') with the product and the difference rounded once (a fused
// multiply-add).  `full` (the same for the whole wave) says that every row of the wave sees every key of the
// tile: then the masks are left out, which changes no bit.  A row that sees no key of the tile keeps its state
// (ca = 1, probabilities 0).
__device__ __forceinline__ void tile_probs(float (&sc)[S_PER_LANE], int kb, int g, bool row_ok, int lo, int pos,
                                           float scale_log2, bool full, float& M, float& L, float& ca,
                                           frag_t (&pf)[KEY_SLABS]) {
  float pr[S_PER_LANE];
  float psum = 0.f;
  float Mn;
  if (full) {
    float tmax = sc[0];
#pragma unroll
    for (int i = 1; i < S_PER_LANE; ++i) tmax = fmaxf(tmax, sc[i]);
    tmax = fmaxf(tmax, lane_xor16(tmax));
    tmax = fmaxf(tmax, lane_xor32(tmax));
    const float m = tmax * scale_log2;
    Mn = (!(M > -INFINITY) || m > M + MAX_STEP) ? m : M;
    ca = fast_exp2(M - Mn);                 // 1 where the maximum stands, 0 for a row whose state was empty
#pragma unroll
    for (int i = 0; i < S_PER_LANE; ++i) {
      pr[i] = fast_exp2(__builtin_fmaf(sc[i], scale_log2, -Mn));
      psum = psum + pr[i];
    }
  } else {
    bool vis[S_PER_LANE];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < S_PER_LANE; ++i) {
      const int key = kb + (i / VK_VEC) * VK_SLAB + g * VK_VEC + (i % VK_VEC);
      vis[i] = row_ok && key >= lo && key <= pos;
      tmax = fmaxf(tmax, vis[i] ? sc[i] : -INFINITY);
    }
    tmax = fmaxf(tmax, lane_xor16(tmax));
    tmax = fmaxf(tmax, lane_xor32(tmax));
    const float m = tmax * scale_log2;      // -inf: the row sees no key of the tile
    Mn = (!(M > -INFINITY) || m > M + MAX_STEP) ? m : M;
    ca = Mn > -INFINITY ? fast_exp2(M - Mn) : 1.f;
#pragma unroll
    for (int i = 0; i < S_PER_LANE; ++i) {
      pr[i] = vis[i] ? fast_exp2(__builtin_fmaf(sc[i], scale_log2, -Mn)) : 0.f;
      psum = psum + pr[i];
    }
  }
  psum = psum + lane_xor16(psum);
  psum = psum + lane_xor32(psum);
  L = __builtin_fmaf(L, ca, psum);
  M = Mn;
#pragma unroll
  for (int ks = 0; ks < KEY_SLABS; ++ks) {
#ifdef VK_BF16
#pragma unroll
    for (int j = 0; j < 8; ++j) pf[ks][j] = (__bf16)pr[ks * 8 + j];
#else
    pf[ks] = f32x4{pr[ks * 4 + 0], pr[ks * 4 + 1], pr[ks * 4 + 2], pr[ks * 4 + 3]};
#endif
  }
}

// ACC * ca, a row's sums so far under its new maximum.  Left out for the wave as a whole when it changes nothing:
// every row's factor is 1 (the maximum stood), or the row's state was empty before this tile (`fresh`: its sums
// are zero).
template <int NDT>
__device__ __forceinline__ void scale_state(f32x4 (&ACC)[NDT], float ca, bool fresh) {
  if (__all(ca == 1.f || fresh)) return;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
    ACC[dt].x = ACC[dt].x * ca;
    ACC[dt].y = ACC[dt].y * ca;
    ACC[dt].z = ACC[dt].z * ca;
    ACC[dt].w = ACC[dt].w * ca;
  }
}

// Keys outside [first, k_len) may lie in pages this sequence does not own
// (never written, or given back once the window passed them): their values
// are replaced by zero so that stale NaN or Inf cannot reach the sum.
__device__ __forceinline__ void zero_unowned(frag_t (&vf)[KEY_SLABS], int kb, int g, int first, int k_len) {
#pragma unroll
  for (int ks = 0; ks < KEY_SLABS; ++ks) {
    const int k0 = kb + ks * VK_SLAB + g * VK_VEC;
#pragma unroll
    for (int j = 0; j < VK_VEC; ++j)
      if (k0 + j >= k_len || k0 + j < first) vf[ks][j] = (elem_t)0.f;
  }
}

// The pieces of a tile's work, for the kernels that read fragments straight from global memory.
// No load is predicated on data: addresses of keys beyond k_len are clamped to a key of this
// sequence (valid memory) and what they bring is masked or zeroed later.  A select on a loaded
// value would make the compiler wait for every load right where it is issued.
constexpr int KSUB = S_PER_LANE / 4;    // 16-key MFMA sub-tiles per tile

// Key fragments of the whole tile, all in flight together.
// EXACT (here and below): the head size is the padded one and a page holds a tile or more, known
// at compile time, so that no branch on either is left in the code.
template <int NQS, bool EXACT>
__device__ __forceinline__ void load_keys(const RowCtx& c, int kb, frag_t (&kf)[KSUB][NQS]) {
  const int d = EXACT ? NQS * VK_SLAB : c.d, P = c.P, lp = c.lp, r16 = c.r16, g = c.g;
  const bool dfull = EXACT || d % VK_SLAB == 0;    // else the last slab along d is partly outside the head
  const int last_key = c.k_len - 1;
  // With pages of at least a tile, the tile lies in one page: one table lookup for the wave.
  const bool one_page = EXACT || P >= TILE_KEYS;
  const elem_t* kpage = c.kbase + (one_page ? (int64_t)c.bt[kb >> lp] * c.page_stride : 0);
#pragma unroll
  for (int sub = 0; sub < KSUB; ++sub) {
#ifdef VK_BF16
    // MFMA row m of sub-tile (ks, u) is key  slab + 8*(m/4) + 4*u + m%4, so that
    // lane group g ends up with the 8 consecutive keys slab + 8g .. 8g+7.
    const int key = kb + (sub >> 1) * VK_SLAB + 8 * (r16 >> 2) + 4 * (sub & 1) + (r16 & 3);
#else
    const int key = kb + sub * VK_SLAB + r16;
#endif
    const int kk = min(key, last_key);
    const elem_t* krow = (one_page ? kpage : c.kbase + c.bt[kk >> lp] * c.page_stride) + (int64_t)(kk & (P - 1)) * d;
#pragma unroll
    for (int s = 0; s < NQS; ++s) {
      if (s * VK_SLAB < d) {
        const int col = s * VK_SLAB + g * VK_VEC;
        kf[sub][s] = dfull ? *reinterpret_cast<const frag_t*>(krow + col) : load_frag(krow + col, col < d);
      }
    }
  }
}

template <int NDT, bool EXACT>
__device__ __forceinline__ void load_values(const RowCtx& c, int kb, frag_t (&vf)[NDT][KEY_SLABS]) {
  const int d = EXACT ? NDT * 16 : c.d, P = c.P, lp = c.lp, r16 = c.r16, g = c.g;
  const int last_key = c.k_len - 1;
  const bool one_page = EXACT || P >= TILE_KEYS;
  const elem_t* vpage = c.vbase + (one_page ? (int64_t)c.bt[kb >> lp] * c.page_stride : 0);
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
    if (dt * 16 < d) {
#pragma unroll
      for (int ks = 0; ks < KEY_SLABS; ++ks) {
        const int k0 = kb + ks * VK_SLAB + g * VK_VEC;
        const int kk = k0 <= last_key ? k0 : kb;     // a whole vector inside a page of this sequence
        const elem_t* vrow = (one_page ? vpage : c.vbase + c.bt[kk >> lp] * c.page_stride) +
                             (int64_t)(dt * 16 + r16) * P + (kk & (P - 1));
        vf[dt][ks] = *reinterpret_cast<const frag_t*>(vrow);
      }
    }
  }
}

// Scores S^T[key, row] = K Q^T.
template <int NQS, bool EXACT>
__device__ __forceinline__ void tile_scores(const RowCtx& c, const frag_t (&kf)[KSUB][NQS], const frag_t (&qf)[NQS],
                                            float (&sc)[S_PER_LANE]) {
  const int d = EXACT ? NQS * VK_SLAB : c.d;
#pragma unroll
  for (int sub = 0; sub < KSUB; ++sub) {
    f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NQS; ++s)
      if (s * VK_SLAB < d) s4 = mma_slab(kf[sub][s], qf[s], s4);
    sc[4 * sub + 0] = s4.x;
    sc[4 * sub + 1] = s4.y;
    sc[4 * sub + 2] = s4.z;
    sc[4 * sub + 3] = s4.w;
  }
}

// ACC += V^T P^T; values of keys the sequence does not own count as zero.
template <int NDT, bool EXACT>
__device__ __forceinline__ void tile_pv(const RowCtx& c, int kb, frag_t (&vf)[NDT][KEY_SLABS], const frag_t (&pf)[KEY_SLABS],
                                        f32x4 (&ACC)[NDT]) {
  const int d = EXACT ? NDT * 16 : c.d;
  if (kb + TILE_KEYS > c.k_len || kb < c.wave_lo) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
      if (dt * 16 < d) zero_unowned(vf[dt], kb, c.g, c.wave_lo, c.k_len);
  }
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
    if (dt * 16 < d) {
#pragma unroll
      for (int ks = 0; ks < KEY_SLABS; ++ks) ACC[dt] = mma_slab(vf[dt][ks], pf[ks], ACC[dt]);
    }
  }
}

// One tile onto the segment's state (M, L, ACC) of this lane's row, fragments straight from global memory.
template <int NDT, int NQS, bool V_LATE, bool EXACT = false>
__device__ __forceinline__ void tile_step(const RowCtx& c, const frag_t (&qf)[NQS], int kb, float& M, float& L,
                                          f32x4 (&ACC)[NDT]) {
  frag_t kf[KSUB][NQS];
  frag_t vf[NDT][KEY_SLABS];
  load_keys<NQS, EXACT>(c, kb, kf);
  // A wave that has the SIMD nearly to itself (few decoded tokens) asks for everything at once.
  if (!V_LATE) load_values<NDT, EXACT>(c, kb, vf);
  float sc[S_PER_LANE];
  tile_scores<NQS, EXACT>(c, kf, qf, sc);
  if (V_LATE) {
    // Requested once the key fragments' registers are free again, so that more waves fit a SIMD;
    // the latency passes behind the softmax arithmetic and the other waves.
    __builtin_amdgcn_sched_barrier(0);
    load_values<NDT, EXACT>(c, kb, vf);
  }
  frag_t pf[KEY_SLABS];
  float ca;
  const bool fresh = !(M > -INFINITY);
  tile_probs(sc, kb, c.g, c.row_ok, c.lo, c.pos, c.scale_log2, false, M, L, ca, pf);
  scale_state<NDT>(ACC, ca, fresh);
  tile_pv<NDT, EXACT>(c, kb, vf, pf, ACC);
}

// state (M, L, ACC) <- fold of a non-empty segment (m, l, acc).
__device__ __forceinline__ void fold_scales(float M, float m, float& Mn, float& ca, float& cb) {
  Mn = fmaxf(M, m);
  ca = fast_exp2(M - Mn);
  cb = fast_exp2(m - Mn);
}
__device__ __forceinline__ float fold1(float A, float a, float ca, float cb) { return __builtin_fmaf(a, cb, A * ca); }

template <int NDT>
__device__ __forceinline__ void fold(float& M, float& L, f32x4 (&ACC)[NDT], float m, float l, const f32x4 (&acc)[NDT]) {
  if (!(m > -INFINITY)) return;
  float Mn, ca, cb;
  fold_scales(M, m, Mn, ca, cb);
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
    ACC[dt].x = fold1(ACC[dt].x, acc[dt].x, ca, cb);
    ACC[dt].y = fold1(ACC[dt].y, acc[dt].y, ca, cb);
    ACC[dt].z = fold1(ACC[dt].z, acc[dt].z, ca, cb);
    ACC[dt].w = fold1(ACC[dt].w, acc[dt].w, ca, cb);
  }
  L = fold1(L, l, ca, cb);
  M = Mn;
}

template <int NQS>
__device__ __forceinline__ void load_q(const AttnArgs& a, int tok, int head, bool row_ok, int g, frag_t (&qf)[NQS]) {
  const elem_t* qrow = a.q + ((int64_t)(row_ok ? tok : 0) * a.nq + (row_ok ? head : 0)) * a.d;
#pragma unroll
  for (int s = 0; s < NQS; ++s) {
    const int col = s * VK_SLAB + g * VK_VEC;
    qf[s] = load_frag(qrow + col, row_ok && col < a.d);
  }
}

__device__ __forceinline__ void init_ctx(RowCtx& c, const AttnArgs& a, int seq, int kvh, int k_len) {
  const int64_t page_elems = (int64_t)a.P * a.d;
  c.bt = a.block_table + (int64_t)seq * a.bt_stride;
  c.kbase = a.kc + (int64_t)kvh * page_elems;
  c.vbase = a.vc + (int64_t)kvh * page_elems;
  c.page_stride = (int64_t)a.nkv * page_elems;
  c.k_len = k_len;
  c.d = a.d;
  c.P = a.P;
  c.lp = __builtin_ctz(a.P);
  c.scale_log2 = a.scale_log2;
}

// Prompt portions, the kernel for every head size and page size: an item is up
// to ITEM_ROWS consecutive rows of one sequence, a workgroup takes 16 of them.
// It has one wave per q head of a kv head (up to 4), so that the waves of a
// group read the same keys and values, straight from global memory, at about
// the same time.
template <int DPAD>
__global__ __launch_bounds__(256) void attn_prefill_kernel(AttnArgs a, int heads_per_wg) {
  constexpr int NDT = DPAD / 16, NQS = DPAD / VK_SLAB;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int G = a.nq / a.nkv;
  const int groups_per_kv = (G + heads_per_wg - 1) / heads_per_wg;
  const int kvh = blockIdx.y / groups_per_kv;
  const int hg = (blockIdx.y - kvh * groups_per_kv) * heads_per_wg + wave;
  if (hg >= G) return;
  const int head = kvh * G + hg;
  const int item = blockIdx.x / (ITEM_ROWS / 16);
  const int seq = a.items[2 * item];
  const int q_off = a.items[2 * item + 1] + (blockIdx.x % (ITEM_ROWS / 16)) * 16;
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  if (q_off >= q_len) return;
  const int k_len = a.k_len[seq];
  RowCtx c;
  init_ctx(c, a, seq, kvh, k_len);
  c.r16 = lane & 15;
  c.g = lane >> 4;
  const int nvalid = min(16, q_len - q_off);
  c.row_ok = c.r16 < nvalid;
  const int tok = q_begin + q_off + c.r16;
  const int pos0 = k_len - q_len + q_off;
  c.pos = pos0 + c.r16;
  c.lo = a.window > 0 ? max(0, c.pos - a.window + 1) : 0;
  c.wave_lo = a.window > 0 ? max(0, pos0 - a.window + 1) : 0;
  const int tile_lo = c.wave_lo / TILE_KEYS, tile_hi = (pos0 + nvalid - 1) / TILE_KEYS;

  frag_t qf[NQS];
  load_q<NQS>(a, tok, head, c.row_ok, c.g, qf);

  float M = -INFINITY, L = 0.f;
  f32x4 ACC[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) ACC[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int seg = tile_lo / SEG_TILES; seg <= tile_hi / SEG_TILES; ++seg) {
    float Ms = -INFINITY, Ls = 0.f;
    f32x4 As[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) As[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int t_end = min(tile_hi, seg * SEG_TILES + SEG_TILES - 1);
    for (int t = max(tile_lo, seg * SEG_TILES); t <= t_end; ++t) tile_step<NDT, NQS, true>(c, qf, t * TILE_KEYS, Ms, Ls, As);
    fold<NDT>(M, L, ACC, Ms, Ls, As);
  }
  if (c.row_ok) {
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    elem_t* orow = a.out + ((int64_t)tok * a.nq + head) * a.d;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      if (dt * 16 < a.d) {
        const float o[4] = {ACC[dt].x * inv, ACC[dt].y * inv, ACC[dt].z * inv, ACC[dt].w * inv};
        elem_t* p = orow + dt * 16 + 4 * c.g;
#pragma unroll
        for (int i = 0; i < 4; ++i) p[i] = from_f32<elem_t>(o[i]);
      }
    }
  }
}

// Prompt portions, the fast kernel: head sizes 64, 128, 256 with pages of at
// least a tile.  A workgroup is one q head and one item; each of its NW waves has
// one 16-row tile of the item's rows.  Every key tile goes from global memory
// straight into LDS once (global_load_lds_dwordx4, two buffers: the next tile
// lands while this one is used) and is read from there by all waves.  A tile's
// work is three stretches of code that the compiler does not mix: the scores
// (key fragments from LDS, MFMAs), the probabilities and the scaling of the
// row's sums (vector instructions), the product with the values (value fragments
// from LDS, MFMAs); a wave runs the two with MFMAs at a raised priority, so that
// of the two waves of a SIMD the one that feeds the matrix unit goes first and the
// other's vector instructions fill in.  The arithmetic per row is tile_step's and
// fold's, operation for operation.
//
// LDS holds the key tile as [64 keys][d] and the value tile as [d][64 keys],
// in 16-byte columns that are XOR-swizzled by row so that the 16 lanes of a
// fragment read hit different banks.  A wave-level load fills 1 KB of LDS in
// lane order, so the swizzle is applied to the global address a lane reads.
__device__ __forceinline__ void wait_vm_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0) only
// 16 bytes per lane from global memory into LDS at dst + 16 * lane (dst is the same for the wave).
__device__ __forceinline__ void load_to_lds16(const elem_t* src, unsigned char* dst) {
  __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
}

#ifdef VK_BF16
// MFMA row r16 of key sub-tile `sub` (see tile_partial) and the swizzle of a key row.
__device__ __forceinline__ int key_row_of(int sub, int r16) { return (sub >> 1) * VK_SLAB + 8 * (r16 >> 2) + 4 * (sub & 1) + (r16 & 3); }
__device__ __forceinline__ int key_swz(int row) { return (((row >> 3) & 3) << 2) | (row & 3); }
__device__ __forceinline__ int val_swz(int row) { return (row >> 1) & 7; }    // rows of 128 bytes
#else
__device__ __forceinline__ int key_row_of(int sub, int r16) { return sub * VK_SLAB + r16; }
__device__ __forceinline__ int key_swz(int row) { return row & 15; }
__device__ __forceinline__ int val_swz(int row) { return row & 15; }          // rows of 256 bytes
#endif

template <int DPAD, int NW, int NST = 2>
__global__ __launch_bounds__(64 * NW, 2) void attn_prefill_lds_kernel(AttnArgs a, int n_items) {
  constexpr int ROWS_WG = 16 * NW;                       // NW waves, each with one 16-row tile
  constexpr int BPI = ITEM_ROWS / ROWS_WG;               // workgroups per item
  static_assert(ITEM_ROWS % ROWS_WG == 0, "a workgroup's rows must divide an item");
  constexpr int NDT = DPAD / 16, NQS = DPAD / VK_SLAB;
  constexpr int EB = (int)sizeof(elem_t);
  constexpr int KRB = DPAD * EB, CK = KRB / 16;          // key row: bytes, 16-byte columns
  constexpr int VRB = TILE_KEYS * EB, CV = VRB / 16;     // value row (one d index, 64 keys)
  constexpr int KT_BYTES = TILE_KEYS * KRB, STAGE = 2 * KT_BYTES;   // value tile: DPAD * VRB, the same
  constexpr int NI = CK / NW;                            // wave-level loads per wave for keys; as many for values
  constexpr int KMASK = CK >= 16 ? 15 : CK - 1;
  static_assert(CK % NW == 0, "head size too small for this kernel");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [2][key tile, value tile]

  // The wave's index as a scalar: what depends on it alone then branches for the wave as a whole.
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  // Workgroup i runs on chip part i % 8, each with a cache of its own.  Long items first (items
  // are in ascending row order and later rows see more keys), dealt to the parts in turn, and the q
  // heads of an item, which share keys, one after the other on the same part.
  const int lin = blockIdx.x;
  const int n_blocks = n_items * BPI;
  int rank, head;            // rank: 0 for the last rows of the last item
  if (n_blocks % 8 == 0) {
    // Rounds of eight ranks; every other round is dealt backwards, so that a part's long and
    // short workgroups add up alike (with two rounds: ranks x and 15 - x on part x).
    const int j = lin >> 3, round = j / a.nq, x = lin & 7;
    rank = round * 8 + ((round & 1) ? 7 - x : x);
    head = j % a.nq;
  } else {
    rank = lin / a.nq;
    head = lin % a.nq;
  }
  const int block = n_blocks - 1 - rank;
  const int item = block / BPI;
  const int kvh = head / (a.nq / a.nkv);
  const int seq = a.items[2 * item], q_off0 = a.items[2 * item + 1] + (block % BPI) * ROWS_WG;
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  if (q_off0 >= q_len) return;                           // the item ends before this workgroup's rows: the whole workgroup
  const int k_len = a.k_len[seq];
  const int rows_item = min(ROWS_WG, q_len - q_off0);    // this workgroup's rows
  const int pos_item = k_len - q_len + q_off0;           // position of the item's first row
  const int item_lo = a.window > 0 ? max(0, pos_item - a.window + 1) : 0;
  const int tile_lo = item_lo / TILE_KEYS, tile_hi = (pos_item + rows_item - 1) / TILE_KEYS;

  // ---- this wave's rows ----
  const int rows_wave = min(16, rows_item - 16 * wave);  // <= 0: the wave only helps to load
  const int pos_wave = pos_item + 16 * wave;
  const int wave_lo = a.window > 0 ? max(0, pos_wave - a.window + 1) : 0;
  const int wtile_lo = wave_lo / TILE_KEYS, wtile_hi = rows_wave > 0 ? (pos_wave + rows_wave - 1) / TILE_KEYS : -1;
  const bool row_ok = r16 < rows_wave;
  const int pos = pos_wave + r16;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int tok = q_begin + q_off0 + 16 * wave + r16;
  frag_t qf[NQS];
  load_q<NQS>(a, tok, head, row_ok, g, qf);

  // ---- what this lane fetches of every tile ----
  const int64_t page_elems = (int64_t)a.P * a.d;
  const elem_t* kbase = a.kc + (int64_t)kvh * page_elems;
  const elem_t* vbase = a.vc + (int64_t)kvh * page_elems;
  const int64_t page_stride = (int64_t)a.nkv * page_elems;
  const int32_t* bt = a.block_table + (int64_t)seq * a.bt_stride;
  const int lp = __builtin_ctz(a.P);
  int koff[NI], voff[NI];       // element offsets from the tile's first key (keys) or from its page row 0 (values)
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int instr = wave + NW * j;                       // 1 KB of the tile each
    const int krow = instr * (1024 / KRB) + lane / CK;     // key within the tile
    const int kcol = (lane % CK) ^ (key_swz(krow) & KMASK);
    koff[j] = krow * DPAD + kcol * VK_VEC;
    const int vrow = instr * (1024 / VRB) + lane / CV;     // index along d
    const int vcol = (lane % CV) ^ val_swz(vrow);
    voff[j] = vrow * a.P + vcol * VK_VEC;
  }
  auto issue = [&](int t, int stage) {
    const int kb = t * TILE_KEYS;
    // The page number is the same for the wave: as a scalar, its arithmetic stays off the vector unit.
    const int64_t page = (int64_t)__builtin_amdgcn_readfirstlane(bt[kb >> lp]) * page_stride;
    const int in_page = kb & (a.P - 1);
    const elem_t* kt = kbase + page + (int64_t)in_page * DPAD;
    const elem_t* vt = vbase + page + in_page;
    unsigned char* dst = lds + stage * STAGE + wave * 1024;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      load_to_lds16(kt + koff[j], dst + j * NW * 1024);
      load_to_lds16(vt + voff[j], dst + KT_BYTES + j * NW * 1024);
    }
  };

  float M = -INFINITY, L = 0.f, Ms = -INFINITY, Ls = 0.f;
  f32x4 ACC[NDT], As[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) ACC[dt] = As[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  issue(tile_lo, 0);
  // The buffer a tile lies in is a constant in the code of its step (the loop below takes two steps a turn), so that
  // the LDS addresses of the fragments are computed once for the kernel and not added to a buffer's base in every tile.
  auto step = [&](int t, auto stage_c) {
    constexpr int stage = decltype(stage_c)::value;
    wait_vm_loads();
    __syncthreads();      // tile t is in LDS; every wave is done with the other buffer
    if (NST == 2 && t < tile_hi) issue(t + 1, stage ^ 1);
    if (t * TILE_KEYS + TILE_KEYS > k_len || t * TILE_KEYS < item_lo) {
      // Keys outside [item_lo, k_len) may lie in pages this sequence does not own: their values are replaced by
      // zero in LDS, so that stale NaN or Inf cannot reach a sum (their probabilities are zero).  The first and
      // the last tile of an item at most; the same for every wave, which all pass the second barrier.
      const int kb = t * TILE_KEYS;
      unsigned char* vt = lds + stage * STAGE + KT_BYTES;
      for (int e = threadIdx.x; e < DPAD * TILE_KEYS; e += 64 * NW) {
        const int vrow = e / TILE_KEYS, key = e % TILE_KEYS;
        if (kb + key >= k_len || kb + key < item_lo) {
          const int col = (key / VK_VEC) ^ val_swz(vrow);
          *reinterpret_cast<elem_t*>(vt + vrow * VRB + col * 16 + (key % VK_VEC) * EB) = (elem_t)0.f;
        }
      }
      __syncthreads();
    }
    if (t >= wtile_lo && t <= wtile_hi) {
      const int kb = t * TILE_KEYS;
      const unsigned char* kl = lds + stage * STAGE;
      const unsigned char* vl = kl + KT_BYTES;
      // ---- scores ----
      float sc[S_PER_LANE];
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int sub = 0; sub < S_PER_LANE / 4; ++sub) {
        const int krow = key_row_of(sub, r16);
        const unsigned char* kr = kl + krow * KRB;
        const int sw = key_swz(krow) & KMASK;
        frag_t kf[NQS];
#pragma unroll
        for (int s = 0; s < NQS; ++s) kf[s] = *reinterpret_cast<const frag_t*>(kr + (((s * 4 + g) ^ sw) << 4));
        f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NQS; ++s) s4 = mma_slab(kf[s], qf[s], s4);
        sc[4 * sub + 0] = s4.x;
        sc[4 * sub + 1] = s4.y;
        sc[4 * sub + 2] = s4.z;
        sc[4 * sub + 3] = s4.w;
      }
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      // ---- the row's new maximum, its probabilities, its sums so far under the new maximum ----
      const bool full = rows_wave >= 16 && kb + TILE_KEYS - 1 <= pos_wave &&
                        kb >= (a.window > 0 ? max(0, pos_wave + 15 - a.window + 1) : 0);
      frag_t pf[KEY_SLABS];
      float ca;
      const bool fresh = !(Ms > -INFINITY);
      tile_probs(sc, kb, g, row_ok, lo, pos, a.scale_log2, full, Ms, Ls, ca, pf);
      scale_state<NDT>(As, ca, fresh);
      __builtin_amdgcn_sched_barrier(0);
      // ---- P V onto the segment's sums, column block by column block ----
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        const int vrow = dt * 16 + r16;
        const unsigned char* vr = vl + vrow * VRB;
        const int sw = val_swz(vrow);
        frag_t vf[KEY_SLABS];
#pragma unroll
        for (int ks = 0; ks < KEY_SLABS; ++ks) vf[ks] = *reinterpret_cast<const frag_t*>(vr + (((ks * 4 + g) ^ sw) << 4));
#pragma unroll
        for (int ks = 0; ks < KEY_SLABS; ++ks) As[dt] = mma_slab(vf[ks], pf[ks], As[dt]);
      }
      __builtin_amdgcn_s_setprio(0);
    }
    if (NST == 1 && t < tile_hi) {                         // one buffer: the next tile may come when every wave has read this one
      __syncthreads();
      issue(t + 1, 0);
    }
    if ((t + 1) % SEG_TILES == 0 || t == tile_hi) {        // the segment is complete
      fold<NDT>(M, L, ACC, Ms, Ls, As);
      Ms = -INFINITY;
      Ls = 0.f;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) As[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  };
  for (int t = tile_lo; t <= tile_hi; t += 2) {
    step(t, std::integral_constant<int, 0>{});
    if (t + 1 <= tile_hi) step(t + 1, std::integral_constant<int, NST == 2 ? 1 : 0>{});
  }
  if (row_ok) {
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    elem_t* orow = a.out + ((int64_t)tok * a.nq + head) * a.d;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const float o[4] = {ACC[dt].x * inv, ACC[dt].y * inv, ACC[dt].z * inv, ACC[dt].w * inv};
      elem_t* op = orow + dt * 16 + 4 * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) op[i] = from_f32<elem_t>(o[i]);
    }
  }
}

// Decoded tokens: an item is one token; the 16 rows of a wave are up to 16 q heads of one kv head.  A wave takes
// a segment, tile after tile, and asks for a tile's fragments when it needs them: for head and element sizes whose
// fragments of two tiles do not fit a wave's registers.  The waves of a workgroup are neighbouring segments.
#define PLAIN_WAVES 4
template <int DPAD, bool V_LATE>
__global__ __launch_bounds__(64 * PLAIN_WAVES) void attn_decode_plain_kernel(AttnArgs a) {
  constexpr int NDT = DPAD / 16, NQS = DPAD / VK_SLAB;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = a.nq / a.nkv, HT = (G + 15) >> 4;
  const int kvh = blockIdx.y / HT, ht = blockIdx.y - kvh * HT;
  const int seg = blockIdx.z * PLAIN_WAVES + wave;
  const int seq = a.items[2 * blockIdx.x], q_off = a.items[2 * blockIdx.x + 1];
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  const int k_len = a.k_len[seq];
  const int tok = q_begin + q_off;
  const int pos = k_len - q_len + q_off;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int t0 = max(lo / TILE_KEYS, seg * SEG_TILES), t1 = min(pos / TILE_KEYS, seg * SEG_TILES + SEG_TILES - 1);
  if (t0 > t1) return;   // whole wave; no barrier follows

  RowCtx c;
  init_ctx(c, a, seq, kvh, k_len);
  c.r16 = lane & 15;
  c.g = lane >> 4;
  c.row_ok = c.r16 < min(16, G - ht * 16);
  c.pos = pos;
  c.lo = lo;
  c.wave_lo = lo;
  const int head = kvh * G + ht * 16 + c.r16;
  frag_t qf[NQS];
  load_q<NQS>(a, tok, head, c.row_ok, c.g, qf);
  float M = -INFINITY, L = 0.f;
  f32x4 ACC[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) ACC[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int t = t0; t <= t1; ++t) tile_step<NDT, NQS, V_LATE>(c, qf, t * TILE_KEYS, M, L, ACC);
  if (!c.row_ok) return;
  const int64_t prow = ((int64_t)blockIdx.x * a.nq + head) * a.nseg + seg;
  if (c.g == 0) {
    a.part_ml[2 * prow] = M;
    a.part_ml[2 * prow + 1] = L;
  }
  if (M > -INFINITY) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
      if (dt * 16 < a.d) *reinterpret_cast<f32x4*>(&a.part_acc[prow * a.d + dt * 16 + 4 * c.g]) = ACC[dt];
  }
}

// Decoded tokens with many keys: a wave takes a whole segment, tile after tile, its state in
// registers.  The keys of the next tile are asked for as soon as this tile's scores have left
// their registers, the next values once this tile's product is done, so that a wave has half a
// tile or more in flight all the time and the tables and the q rows are read once per segment.
// No LDS and no barrier; the waves of a workgroup are neighbouring segments.
#define SEG_WAVES 2
template <int DPAD, bool EXACT>
__global__ __launch_bounds__(64 * SEG_WAVES, 2) void attn_decode_seg_kernel(AttnArgs a) {
  constexpr int NDT = DPAD / 16, NQS = DPAD / VK_SLAB;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = a.nq / a.nkv, HT = (G + 15) >> 4;
  const int kvh = blockIdx.y / HT, ht = blockIdx.y - kvh * HT;
  const int seg = blockIdx.z * SEG_WAVES + wave;
  const int seq = a.items[2 * blockIdx.x], q_off = a.items[2 * blockIdx.x + 1];
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  const int k_len = a.k_len[seq];
  const int tok = q_begin + q_off;
  const int pos = k_len - q_len + q_off;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int t0 = max(lo / TILE_KEYS, seg * SEG_TILES), t1 = min(pos / TILE_KEYS, seg * SEG_TILES + SEG_TILES - 1);
  if (t0 > t1) return;   // whole wave; no barrier follows

  RowCtx c;
  init_ctx(c, a, seq, kvh, k_len);
  c.r16 = lane & 15;
  c.g = lane >> 4;
  c.row_ok = c.r16 < min(16, G - ht * 16);
  c.pos = pos;
  c.lo = lo;
  c.wave_lo = lo;
  const int head = kvh * G + ht * 16 + c.r16;
  frag_t qf[NQS];
  load_q<NQS>(a, tok, head, c.row_ok, c.g, qf);
  frag_t kf[KSUB][NQS];
  frag_t vf[NDT][KEY_SLABS];
  load_keys<NQS, EXACT>(c, t0 * TILE_KEYS, kf);
  load_values<NDT, EXACT>(c, t0 * TILE_KEYS, vf);
  float M = -INFINITY, L = 0.f;
  f32x4 ACC[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) ACC[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto tile = [&](int t, bool more) {
    const int kb = t * TILE_KEYS;
    float sc[S_PER_LANE];
    tile_scores<NQS, EXACT>(c, kf, qf, sc);
    __builtin_amdgcn_sched_barrier(0);
    if (more) load_keys<NQS, EXACT>(c, kb + TILE_KEYS, kf);
    __builtin_amdgcn_sched_barrier(0);
    // Every row of a decoded token's wave stands at the same position: the masks are needed in the
    // tiles that hold the window's edge or the token itself only.
    const bool full = kb >= lo && kb + TILE_KEYS - 1 <= pos;
    frag_t pf[KEY_SLABS];
    float ca;
    const bool fresh = !(M > -INFINITY);
    tile_probs(sc, kb, c.g, c.row_ok, lo, pos, c.scale_log2, full, M, L, ca, pf);
    scale_state<NDT>(ACC, ca, fresh);
    tile_pv<NDT, EXACT>(c, kb, vf, pf, ACC);
    __builtin_amdgcn_sched_barrier(0);
    if (more) load_values<NDT, EXACT>(c, kb + TILE_KEYS, vf);
    __builtin_amdgcn_sched_barrier(0);
  };
  // The last tile apart, so that the loop's body has no branch around its loads and the compiler
  // counts the loads in flight exactly.
  for (int t = t0; t < t1; ++t) tile(t, true);
  tile(t1, false);
  if (!c.row_ok) return;
  const int64_t prow = ((int64_t)blockIdx.x * a.nq + head) * a.nseg + seg;
  if (c.g == 0) {
    a.part_ml[2 * prow] = M;
    a.part_ml[2 * prow + 1] = L;
  }
  if (M > -INFINITY) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
      if (EXACT || dt * 16 < a.d) *reinterpret_cast<f32x4*>(&a.part_acc[prow * a.d + dt * 16 + 4 * c.g]) = ACC[dt];
  }
}

// The same with two waves a segment, for steps with so few (token, kv head, segment) triples that a wave each
// leaves most of the chip idle and every wave waits for its four tiles one after the other: the first wave
// takes the first half of the segment's tiles, the second wave the rest.  The second wave asks for its first
// tile's keys and values at once and computes that tile's scores, which need no state; when the first wave has
// left the segment's state in LDS, the second takes it and goes on from there as the one wave would: the same
// bits, and the loads of both halves in flight together.
template <int DPAD, bool EXACT>
__global__ __launch_bounds__(128, 2) void attn_decode_pair_kernel(AttnArgs a) {
  constexpr int NDT = DPAD / 16, NQS = DPAD / VK_SLAB;
  __shared__ f32x4 hand_acc[NDT][64];
  __shared__ float hand_ml[2][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = a.nq / a.nkv, HT = (G + 15) >> 4;
  const int kvh = blockIdx.y / HT, ht = blockIdx.y - kvh * HT;
  const int seg = blockIdx.z;
  const int seq = a.items[2 * blockIdx.x], q_off = a.items[2 * blockIdx.x + 1];
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  const int k_len = a.k_len[seq];
  const int tok = q_begin + q_off;
  const int pos = k_len - q_len + q_off;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int s0 = max(lo / TILE_KEYS, seg * SEG_TILES), s1 = min(pos / TILE_KEYS, seg * SEG_TILES + SEG_TILES - 1);
  if (s0 > s1) return;                                  // the whole workgroup
  const int n = s1 - s0 + 1, n_first = (n + 1) >> 1;
  const bool paired = n > 1;                            // the same for both waves
  const int t0 = wave == 0 ? s0 : s0 + n_first, t1 = wave == 0 ? s0 + n_first - 1 : s1;
  if (t0 > t1) return;                                  // the second wave of a segment with one tile: no barrier follows for the first either

  RowCtx c;
  init_ctx(c, a, seq, kvh, k_len);
  c.r16 = lane & 15;
  c.g = lane >> 4;
  c.row_ok = c.r16 < min(16, G - ht * 16);
  c.pos = pos;
  c.lo = lo;
  c.wave_lo = lo;
  const int head = kvh * G + ht * 16 + c.r16;
  frag_t qf[NQS];
  load_q<NQS>(a, tok, head, c.row_ok, c.g, qf);
  frag_t kf[KSUB][NQS];
  frag_t vf[NDT][KEY_SLABS];
  load_keys<NQS, EXACT>(c, t0 * TILE_KEYS, kf);
  load_values<NDT, EXACT>(c, t0 * TILE_KEYS, vf);
  float M = -INFINITY, L = 0.f;
  f32x4 ACC[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) ACC[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float sc[S_PER_LANE];
  // A tile's scores, and its successor's keys asked for.
  auto front = [&](int t, bool more) {
    tile_scores<NQS, EXACT>(c, kf, qf, sc);
    __builtin_amdgcn_sched_barrier(0);
    if (more) load_keys<NQS, EXACT>(c, (t + 1) * TILE_KEYS, kf);
    __builtin_amdgcn_sched_barrier(0);
  };
  // The tile onto the state, and its successor's values asked for.
  auto back = [&](int t, bool more) {
    const int kb = t * TILE_KEYS;
    const bool full = kb >= lo && kb + TILE_KEYS - 1 <= pos;
    frag_t pf[KEY_SLABS];
    float ca;
    const bool fresh = !(M > -INFINITY);
    tile_probs(sc, kb, c.g, c.row_ok, lo, pos, c.scale_log2, full, M, L, ca, pf);
    scale_state<NDT>(ACC, ca, fresh);
    tile_pv<NDT, EXACT>(c, kb, vf, pf, ACC);
    __builtin_amdgcn_sched_barrier(0);
    if (more) load_values<NDT, EXACT>(c, kb + TILE_KEYS, vf);
    __builtin_amdgcn_sched_barrier(0);
  };
  // At most two tiles a wave.
  front(t0, t0 < t1);
  if (wave == 1) {
    // The segment's state as the first wave left it (every lane its own part: the same lanes hold the same rows
    // and columns in both waves).
    __syncthreads();
    M = hand_ml[0][lane];
    L = hand_ml[1][lane];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) ACC[dt] = hand_acc[dt][lane];
  }
  back(t0, t0 < t1);
  if (t0 < t1) {
    front(t1, false);
    back(t1, false);
  }
  if (wave == 0 && paired) {
    hand_ml[0][lane] = M;
    hand_ml[1][lane] = L;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) hand_acc[dt][lane] = ACC[dt];
    __syncthreads();
    return;
  }
  if (!c.row_ok) return;
  const int64_t prow = ((int64_t)blockIdx.x * a.nq + head) * a.nseg + seg;
  if (c.g == 0) {
    a.part_ml[2 * prow] = M;
    a.part_ml[2 * prow + 1] = L;
  }
  if (M > -INFINITY) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
      if (EXACT || dt * 16 < a.d) *reinterpret_cast<f32x4*>(&a.part_acc[prow * a.d + dt * 16 + 4 * c.g]) = ACC[dt];
  }
}

// Folds the segment results of one (token, head) in ascending segment order.
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
  float M = -INFINITY, L = 0.f;
  float ACC[4] = {0.f, 0.f, 0.f, 0.f};   // d <= 256
  const int64_t row0 = ((int64_t)blockIdx.x * a.nq + head) * a.nseg;
  // Four segments are fetched together, then folded one after the other.
  for (int seg0 = seg_begin; seg0 < seg_end; seg0 += 4) {
    float m[4], l[4], v[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool in = seg0 + j < seg_end;
      const int64_t r = row0 + (in ? seg0 + j : seg_begin);
      m[j] = in ? a.part_ml[2 * r] : -INFINITY;
      l[j] = a.part_ml[2 * r + 1];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t r = row0 + (seg0 + j < seg_end ? seg0 + j : seg_begin);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int col = threadIdx.x + 64 * i;
        v[j][i] = (col < d && m[j] > -INFINITY) ? a.part_acc[r * d + col] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (m[j] > -INFINITY) {
        float Mn, ca, cb;
        fold_scales(M, m[j], Mn, ca, cb);
#pragma unroll
        for (int i = 0; i < 4; ++i) ACC[i] = fold1(ACC[i], v[j][i], ca, cb);
        L = fold1(L, l[j], ca, cb);
        M = Mn;
      }
    }
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  elem_t* orow = a.out + ((int64_t)tok * a.nq + head) * d;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int col = threadIdx.x + 64 * i;
    if (col < d) orow[col] = from_f32<elem_t>(ACC[i] * inv);
  }
}

extern "C" {

// Number of floats of scratch a decode launch needs for `items` decoded tokens (mode 1 items; the
// prompt rows of the same step need none).
int64_t vk_attn_scratch_floats(int items, int nq, int d, int nseg) {
  const int64_t rows = (int64_t)items * nq * nseg;
  return ((rows * 2 + 3) & ~(int64_t)3) + rows * d;
}

int vk_attn_segment_keys(void) { return TILE_KEYS * SEG_TILES; }

int vk_attn_item_rows(void) { return ITEM_ROWS; }

static int vk_dpad(int d) { return d <= 64 ? 64 : (d <= 128 ? 128 : 256); }

static int attn_device_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (cus <= 0) cus = 256;
  }
  return cus;
}

// 1 if prompt rows of this shape go through the kernel that shares key tiles in LDS.
int vk_attn_prefill_shares_tiles(int d, int P) {
  return (d == 64 || d == 128 || d == 256) && P >= TILE_KEYS && 4 * TILE_KEYS * d * (int)sizeof(elem_t) <= 128 * 1024;
}

// items: n_items pairs (sequence, first row).
// mode 0: each item is up to vk_attn_item_rows() consecutive rows of the sequence's q_len new tokens;
//   the kernel is chosen by shape.  mode 2: the same through the kernel that takes every shape,
//   modes 6, 8 and 9: through the one that shares tiles in LDS with four waves, with eight, and with four and
//   one buffer instead of two, whatever the shape (tests and measurements; the result is the same bits).
// mode 1: each item is one token; the keys are split by segment over nseg workgroups (nseg must cover
//   the longest sequence; scratch must hold vk_attn_scratch_floats(n_items, ...)) and folded by a
//   second kernel; the kernel is chosen by shape.  modes 3, 4, 5, 7: the same through a named kernel
//   (3 and 4: a wave per segment that asks for a tile's fragments when it needs them, the kernel for every
//   shape; 5: a wave per segment with two tiles' fragments in registers; 7: two waves per segment; tests
//   and measurements; the same bits).
int vk_paged_attention(elem_t* out, const elem_t* q, const elem_t* kc, const elem_t* vc,
                       const int32_t* block_table, int bt_stride, const int32_t* cu_q, const int32_t* k_len,
                       const int32_t* items, int n_items, int mode, int nseg, float* scratch, int total_tokens,
                       int nq, int nkv, int d, int P, int window, float scale, hipStream_t st) {
  VK_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "attention: %d q heads are not a multiple of %d kv heads", nq, nkv);
  VK_REQUIRE(d >= 16 && d <= 256 && d % 16 == 0, "attention: head size %d must be a multiple of 16 in 16..256", d);
  VK_REQUIRE(P >= 8 && (P & (P - 1)) == 0, "attention: page size %d must be a power of two >= 8", P);
  VK_REQUIRE(window >= 0, "attention: window %d must not be negative", window);
  VK_REQUIRE(scale > 0.f, "attention: the score scale must be positive");
  VK_REQUIRE(mode >= 0 && mode <= 9, "attention: unknown mode %d", mode);
  const int vk_prefill_variant = mode == 6 ? 14 : (mode == 8 ? 18 : (mode == 9 ? 19 : 0));
  const int vk_decode_variant = mode == 3 ? 1 : (mode == 4 ? 2 : (mode == 5 ? 3 : (mode == 7 ? 4 : 0)));
  if (mode == 6 || mode == 8 || mode == 9) mode = 0;
  if (mode >= 3) mode = 1;
  if (n_items <= 0) return 0;
  AttnArgs a;
  a.q = q; a.out = out; a.kc = kc; a.vc = vc; a.block_table = block_table; a.cu_q = cu_q; a.k_len = k_len;
  a.items = items; a.bt_stride = bt_stride; a.nq = nq; a.nkv = nkv; a.d = d; a.P = P; a.window = window;
  a.nseg = nseg; a.scale_log2 = scale * 1.4426950408889634f;
  a.part_ml = nullptr; a.part_acc = nullptr;
  const int G = nq / nkv;
  if (mode == 0 && vk_attn_prefill_shares_tiles(d, P)) {
    VK_REQUIRE((int64_t)n_items * (ITEM_ROWS / 16) * nq < (1ll << 31), "attention: too many prompt items");
    const size_t smem = (size_t)4 * TILE_KEYS * d * sizeof(elem_t);
#define PREFILL_LDS(DP, NW)                                                                          \
  do {                                                                                               \
    static bool raised = false;                                                                      \
    if (!raised) {                                                                                   \
      (void)hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<DP, NW>,                        \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);             \
      raised = true;                                                                                 \
    }                                                                                                \
    attn_prefill_lds_kernel<DP, NW><<<n_items * (ITEM_ROWS / (16 * NW)) * nq, 64 * NW, smem, st>>>(a, n_items); \
  } while (0)
#define PREFILL_LDS1(DP)                                                                             \
  do {                                                                                               \
    static bool raised = false;                                                                      \
    if (!raised) {                                                                                   \
      (void)hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<DP, 4, 1>,                      \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);              \
      raised = true;                                                                                 \
    }                                                                                                \
    attn_prefill_lds_kernel<DP, 4, 1><<<n_items * (ITEM_ROWS / 64) * nq, 256, smem / 2, st>>>(a, n_items); \
  } while (0)
    // Eight waves of one row tile each measured best (MI355X, head size 128) unless they are few: with fewer
    // workgroups of eight waves than one and a half per compute unit, workgroups of four waves, twice as many,
    // fill the units better (3 prompts of 300 tokens, 32 heads: 49 -> 43 us; 2 of 1,000 tokens, 8 heads of 64:
    // 83 -> 74; from two workgroups per unit on eight waves win by 2 to 8 %).  Two row tiles per wave would
    // halve the LDS traffic but need more than the 256 registers that two waves per SIMD leave: with spills
    // or with one wave per SIMD they measured 40 % slower.
    const int v = (vk_prefill_variant == 14 || (vk_prefill_variant == 0 && 2 * (int64_t)n_items * nq < 3 * (int64_t)attn_device_cus())) ? 14 : 0;
    // With many workgroups (two rounds or more of the three four-wave workgroups that a compute unit holds when
    // each has one buffer of 32 KB) the occupancy is worth more than loads that overlap a workgroup's own work:
    // 12 waves a unit instead of 8 (2 prompts of 2,048 tokens: 140 -> 121 us; 8,192 tokens: 890 -> 718, with 64
    // heads 1,580 -> 1,388).  With fewer it loses to the rounds (2,048 rows after 14,336 keys: 756 -> 825).
    const bool one_buffer = vk_prefill_variant == 19 ||
                            (vk_prefill_variant == 0 && sizeof(elem_t) == 2 && (int64_t)n_items * nq >= 3 * (int64_t)attn_device_cus());
    if (one_buffer) {
      if (d == 64) PREFILL_LDS1(64); else if (d == 128) PREFILL_LDS1(128); else PREFILL_LDS1(256);
      return vk_check_launch("attention (prompt rows, shared tiles, one buffer)");
    }
    if (d == 64) { if (v == 14) PREFILL_LDS(64, 4); else PREFILL_LDS(64, 8); }
    else if (d == 128) { if (v == 14) PREFILL_LDS(128, 4); else PREFILL_LDS(128, 8); }
    else { if (v == 14) PREFILL_LDS(256, 4); else PREFILL_LDS(256, 8); }
#undef PREFILL_LDS
#undef PREFILL_LDS1
    return vk_check_launch("attention (prompt rows, shared tiles)");
  }
  if (mode != 1) {
    const int hpw = G < 4 ? G : 4;
    VK_REQUIRE((int64_t)n_items * (ITEM_ROWS / 16) < (1ll << 31), "attention: too many prompt items");
    const dim3 grid(n_items * (ITEM_ROWS / 16), nkv * ((G + hpw - 1) / hpw));
    VK_REQUIRE(grid.y <= 65535, "attention: too many heads");
    if (d <= 64) attn_prefill_kernel<64><<<grid, 64 * hpw, 0, st>>>(a, hpw);
    else if (d <= 128) attn_prefill_kernel<128><<<grid, 64 * hpw, 0, st>>>(a, hpw);
    else attn_prefill_kernel<256><<<grid, 64 * hpw, 0, st>>>(a, hpw);
    return vk_check_launch("attention (prompt rows)");
  }
  VK_REQUIRE(nseg > 0 && nseg <= 65535 && scratch != nullptr, "attention: decode needs nseg in 1..65535 and scratch");
  // A wave per segment with the next tile's fragments in flight where a wave's registers hold two tiles'
  // fragments (a tile's keys, or its values, are 32 * head size * element size bytes of them); the kernel that
  // asks for a tile's fragments when it needs them is for the larger head and element sizes.
  const bool seg_fits = sizeof(elem_t) * vk_dpad(d) <= 256;
  a.part_ml = scratch;
  a.part_acc = scratch + (((int64_t)n_items * nq * nseg * 2 + 3) & ~(int64_t)3);
  const dim3 grid(n_items, nkv * ((G + 15) / 16), nseg);
  VK_REQUIRE(grid.y <= 65535 && nq <= 65535, "attention: too many heads");
  static_assert(SEG_TILES == 4, "the pair kernel gives a wave two tiles at most");
  // Two waves a segment while there are no more segments in work than one and a quarter per compute unit
  // (measured on MI355X, head size 128, 8 kv heads, with the fold of the segments; a wave against two waves a
  // segment: 1 token of 2,090 keys, 72 segments, 14.7 against 12.6 us; 2 tokens, 144: 14.9, 12.9; 4 tokens, 288:
  // 15.7, 14.9; 8 tokens of 1,000 keys, 256: 14.0, 13.1; 6 tokens of 2,090, 432: 17.5, 19.2; 8 tokens, 576: 19.8,
  // 21.4; 1 token of 32,800 keys, 1,032: 60.3, 62.0).
  const bool pair_fits = seg_fits;
  if (vk_decode_variant == 4 ||
      (vk_decode_variant == 0 && pair_fits && 4 * (int64_t)grid.x * grid.y * grid.z <= 5 * (int64_t)attn_device_cus())) {
    const bool exact = P >= TILE_KEYS && d == vk_dpad(d);
#define DECODE_PAIR(DP)                                                           \
  do {                                                                            \
    if (exact) attn_decode_pair_kernel<DP, true><<<grid, 128, 0, st>>>(a);        \
    else attn_decode_pair_kernel<DP, false><<<grid, 128, 0, st>>>(a);             \
  } while (0)
    if (d <= 64) DECODE_PAIR(64);
    else if (d <= 128) DECODE_PAIR(128);
    else DECODE_PAIR(256);
#undef DECODE_PAIR
    if (vk_check_launch("attention (decoded rows, two waves per segment)")) return 1;
    attn_combine_kernel<<<dim3(n_items, nq), 64, 0, st>>>(a);
    return vk_check_launch("attention (combine)");
  }
  if (vk_decode_variant == 3 || (vk_decode_variant == 0 && seg_fits)) {
    const bool exact = P >= TILE_KEYS && d == vk_dpad(d);
    const dim3 sgrid(grid.x, grid.y, (nseg + SEG_WAVES - 1) / SEG_WAVES);
#define DECODE_SEG(DP)                                                                     \
  do {                                                                                     \
    if (exact) attn_decode_seg_kernel<DP, true><<<sgrid, 64 * SEG_WAVES, 0, st>>>(a);      \
    else attn_decode_seg_kernel<DP, false><<<sgrid, 64 * SEG_WAVES, 0, st>>>(a);           \
  } while (0)
    if (d <= 64) DECODE_SEG(64);
    else if (d <= 128) DECODE_SEG(128);
    else DECODE_SEG(256);
#undef DECODE_SEG
    if (vk_check_launch("attention (decoded rows, wave per segment)")) return 1;
    attn_combine_kernel<<<dim3(n_items, nq), 64, 0, st>>>(a);
    return vk_check_launch("attention (combine)");
  }
  // With few waves a wave asks for keys and values together; with many, the values wait until the keys'
  // registers are free, so that more waves fit a SIMD.
  const dim3 pgrid(grid.x, grid.y, (nseg + PLAIN_WAVES - 1) / PLAIN_WAVES);
  const bool late = (int64_t)grid.x * grid.y * grid.z > 1024;
#define DECODE_PLAIN(DP)                                                                    \
  do {                                                                                      \
    if (late) attn_decode_plain_kernel<DP, true><<<pgrid, 64 * PLAIN_WAVES, 0, st>>>(a);    \
    else attn_decode_plain_kernel<DP, false><<<pgrid, 64 * PLAIN_WAVES, 0, st>>>(a);        \
  } while (0)
  if (d <= 64) DECODE_PLAIN(64);
  else if (d <= 128) DECODE_PLAIN(128);
  else DECODE_PLAIN(256);
#undef DECODE_PLAIN
  if (vk_check_launch("attention (decoded rows)")) return 1;
  attn_combine_kernel<<<dim3(n_items, nq), 64, 0, st>>>(a);
  return vk_check_launch("attention (combine)");
}

}  // extern "C"
