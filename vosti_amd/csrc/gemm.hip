// out[M,N] = act[M,K] * w[N,K]^T  (weights in [out_features, in_features] layout).
//
// Reduction order, the same in every kernel of this file and for every M:
//   K is cut into chunks of 512 elements starting at 0.  Within a chunk the
//   products are accumulated from zero by mma_slab() over the chunk's slabs in
//   ascending order (weights are the first MFMA operand, activations the
//   second).  The chunk sums are then added to a zero total in ascending chunk
//   order, and the total is rounded to the element type once.
// An output element therefore never depends on M, on the other rows of its
// tile or on which kernel produced it; the choice between the kernels is a
// matter of speed only.  The reference keys its tile configuration on (N, K)
// for the same reason (kernels/triton_kernels/matmul.py:33-73,
// kernels/triton_kernels/qkv_matmul.py:24-32).
//
//   gemm_stream         M <= 64, K a multiple of 512.  Streams the weights once from HBM: persistent
//                       workgroups walk over 16-row weight tiles (one or two at a time); wave w of a
//                       workgroup's W waves takes the chunks w, w+W, ... and keeps a rolling window of
//                       slabs in flight, also across tile borders.  After each round of W chunks the chunk
//                       sums meet in LDS and are added in chunk order.  W is eight, or, up to 16 rows, the
//                       number of chunks where that is 2, 4, 5, 6, 10 or 12 (stream_waves).
//   gemm_stream_swiglu  the same for the gate/up projection with SwiGLU folded in (M <= 16).
//   gemm_mid            17 <= M <= 64, K a multiple of 512: 64 or 32 weight rows per workgroup, weights
//                       streamed into registers, the activations of the chunks in work shared through LDS.
//   gemm_split          M <= 64, K a multiple of 512, 16-bit elements, with a workspace: a workgroup per
//                       (128 weight rows, chunk) leaves its chunk sums in the workspace, a second kernel
//                       adds them in chunk order (vk_gemm_split; vk_gemm_split_preferred says when).
//   gemm_skinny         M <= 64, any K: the same decomposition with predicated loads.
//   gemm_pipe           any M, K a multiple of two slabs (128 bytes of a row): 128x128 output tile per
//                       workgroup, 64x64 per wave, tiles straight from global memory into LDS, two
//                       stages; a second accumulator set holds the total.  Optionally SwiGLU in the
//                       epilogue.
//   gemm_tiled          any M and K: the same tile through registers into LDS, predicated.
#include <cmath>

#include "common.h"
#include "mma.h"
#include "vec.h"

#define KC 512                        // elements per chunk
#define KC_SLABS (KC / VK_SLAB)       // 16 (bfloat16) or 32 (float)
#define SK_WAVES 8

static int device_cus();      // compute units of the current device (defined with the host code below)

__device__ __forceinline__ void store_out4(elem_t* out, int64_t ldo, int m, int n, int M, int N, f32x4 v,
                                           bool vec_ok) {
  if (m >= M || n >= N) return;
  elem_t* p = out + (int64_t)m * ldo + n;
  if (vec_ok && n + 3 < N) {
#ifdef VK_F32
    *reinterpret_cast<f32x4*>(p) = v;
#else
    bf16x4 o;
    o[0] = (__bf16)v.x; o[1] = (__bf16)v.y; o[2] = (__bf16)v.z; o[3] = (__bf16)v.w;
    *reinterpret_cast<bf16x4*>(p) = o;
#endif
  } else {
    p[0] = from_f32<elem_t>(v.x);
    if (n + 1 < N) p[1] = from_f32<elem_t>(v.y);
    if (n + 2 < N) p[2] = from_f32<elem_t>(v.z);
    if (n + 3 < N) p[3] = from_f32<elem_t>(v.w);
  }
}

// ------------------------------------------------------------------ skinny
// MT: 16-row activation tiles (M <= 16*MT).  W: slabs in flight per wave.
template <int MT, int W>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_skinny_kernel(elem_t* __restrict__ out,
                                                                    const elem_t* __restrict__ act,
                                                                    const elem_t* __restrict__ w, int M, int N, int K,
                                                                    int64_t lda, int64_t ldo, int out_vec_ok) {
  static_assert(KC_SLABS % W == 0, "the window must divide a chunk");
  __shared__ f32x4 part[SK_WAVES][MT][64];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int nchunks = (K + KC - 1) / KC;
  const int rounds = (nchunks + SK_WAVES - 1) / SK_WAVES;

  const bool wok = n0 + r16 < N;
  const elem_t* wrow = w + (int64_t)(wok ? n0 + r16 : 0) * K + kg * VK_VEC;
  const elem_t* arow[MT];
  bool aok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r16;
    aok[mt] = m < M;
    arow[mt] = act + (int64_t)(aok[mt] ? m : 0) * lda + kg * VK_VEC;
  }

  frag_t wbuf[W], abuf[W][MT];
  auto issue = [&](int c, int s, int slot) {
    const int k = c * KC + s * VK_SLAB;
    const bool kok = k + kg * VK_VEC < K;
    wbuf[slot] = load_frag(wrow + k, wok && kok);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) abuf[slot][mt] = load_frag(arow[mt] + k, aok[mt] && kok);
  };

  int c = wave;
  if (c < nchunks) {
#pragma unroll
    for (int i = 0; i < W; ++i) issue(c, i, i);
  }
  f32x4 total = {0.f, 0.f, 0.f, 0.f};
  for (int round = 0; round < rounds; ++round, c += SK_WAVES) {
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < nchunks) {
      const int cn = c + SK_WAVES;
      const bool has_next = cn < nchunks;
#pragma unroll
      for (int i = 0; i < KC_SLABS; ++i) {
        const int slot = i % W;
        const frag_t fw = wbuf[slot];
        frag_t fa[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) fa[mt] = abuf[slot][mt];
        if (i + W < KC_SLABS) issue(c, i + W, slot);
        else if (has_next) issue(cn, i + W - KC_SLABS, slot);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] = mma_slab(fw, fa[mt], acc[mt]);
      }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) part[wave][mt][lane] = acc[mt];
    __syncthreads();
    if (wave < MT) {
      for (int w2 = 0; w2 < SK_WAVES; ++w2) {
        if (round * SK_WAVES + w2 < nchunks) {
          const f32x4 p = part[w2][wave][lane];
          total.x = total.x + p.x; total.y = total.y + p.y; total.z = total.z + p.z; total.w = total.w + p.w;
        }
      }
    }
    __syncthreads();
  }
  if (wave < MT) store_out4(out, ldo, wave * 16 + r16, n0 + 4 * kg, M, N, total, out_vec_ok);
}

// ---------------------------------------------------------------- streaming
// The skinny kernel for K a multiple of 512, built to keep HBM busy: workgroups
// are persistent and walk over weight tiles (16 rows) with a stride of the grid;
// a wave's window of W slabs in flight runs on across tile borders, so the
// memory pipe never drains; no load is predicated (rows beyond N or M are
// clamped to the last valid row and their results dropped), because a select on
// a loaded value makes the compiler wait for it at once; and with RC > 0 a wave
// keeps the activations of its RC chunks (K <= RC * 4096) in registers for the
// whole kernel.  One barrier per round of eight chunks.
template <int MT, int W, int RC, int NT, int NW = SK_WAVES>
__global__ __launch_bounds__(64 * NW) void gemm_stream_kernel(elem_t* __restrict__ out,
                                                                    const elem_t* __restrict__ act,
                                                                    const elem_t* __restrict__ w, int M, int N, int K,
                                                                    int64_t lda, int64_t ldo, int out_vec_ok) {
  // NT: 16-row weight tiles per workgroup.  With several activation tiles every workgroup reads all
  // activations once, M * K elements beside its 16 * NT * K weights: more weight rows per workgroup
  // keep that traffic, which comes from the second-level cache, in proportion.
  static_assert(KC_SLABS % W == 0, "the window must divide a chunk");
  // RC: chunks per wave whose activations stay in registers for the whole kernel (0: none are kept;
  // K <= RC * 8 chunks).  A chunk of one activation tile is 64 registers of 16-bit elements.
  constexpr bool RES = RC > 0;
  static_assert(RC * MT <= 2, "resident activations: at most two chunk tiles per wave");
  static_assert(NT * MT <= NW, "one wave adds up each output tile");
  __shared__ f32x4 part[2][NW][NT * MT][64];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int nchunks = K / KC;
  const int ntiles = (N + 16 * NT - 1) / (16 * NT);     // tile: NT * 16 weight rows

  const elem_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) arow[mt] = act + (int64_t)min(mt * 16 + r16, M - 1) * lda + kg * VK_VEC;

  frag_t wbuf[W][NT], abuf[RES ? RC * KC_SLABS : W][MT];
  if (RES) {
#pragma unroll
    for (int r = 0; r < RC; ++r) {
      const int c = min(r * NW + wave, nchunks - 1);     // beyond K: the last chunk again (not used)
#pragma unroll
      for (int s = 0; s < KC_SLABS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          abuf[r * KC_SLABS + s][mt] = *reinterpret_cast<const frag_t*>(arow[mt] + c * KC + s * VK_SLAB);
    }
  }
  auto issue = [&](int tile, int c, int s, int slot) {
    const int k = c * KC + s * VK_SLAB;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      wbuf[slot][nt] = *reinterpret_cast<const frag_t*>(w + (int64_t)min((tile * NT + nt) * 16 + r16, N - 1) * K + kg * VK_VEC + k);
    if (!RES) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) abuf[slot][mt] = *reinterpret_cast<const frag_t*>(arow[mt] + k);
    }
  };

  int tile = blockIdx.x;
  if (tile < ntiles && wave < nchunks) {
#pragma unroll
    for (int i = 0; i < W; ++i) issue(tile, wave, i, i);
  }
  int parity = 0;
  for (; tile < ntiles; tile += gridDim.x) {
    f32x4 total = {0.f, 0.f, 0.f, 0.f};
    auto round = [&](int base, int r) {       // chunks base .. base + 7; r = base / 8 where that is a constant
      const int c = base + wave;
      f32x4 acc[NT][MT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (c < nchunks) {
        // What this wave streams next: its next chunk of this tile, else its first chunk of the next tile.
        int nt_ = tile, nc = c + NW;
        if (nc >= nchunks) {
          nt_ = tile + gridDim.x;
          nc = wave;
        }
        const bool has_next = nt_ < ntiles;
#pragma unroll
        for (int i = 0; i < KC_SLABS; ++i) {
          const int slot = i % W;
          frag_t fw[NT], fa[MT];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) fw[nt] = wbuf[slot][nt];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) fa[mt] = RES ? abuf[r * KC_SLABS + i][mt] : abuf[slot][mt];
          if (i + W < KC_SLABS) issue(tile, c, i + W, slot);
          else if (has_next) issue(nt_, nc, i + W - KC_SLABS, slot);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = mma_slab(fw[nt], fa[mt], acc[nt][mt]);
        }
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) part[parity][wave][nt * MT + mt][lane] = acc[nt][mt];
      __syncthreads();
      if (wave < NT * MT) {
        for (int w2 = 0; w2 < NW; ++w2) {
          if (base + w2 < nchunks) {
            const f32x4 p = part[parity][w2][wave][lane];
            total.x = total.x + p.x; total.y = total.y + p.y; total.z = total.z + p.z; total.w = total.w + p.w;
          }
        }
      }
      parity ^= 1;
    };
    if (RES) {
#pragma unroll
      for (int r = 0; r < (RES ? RC : 1); ++r)
        if (r * NW < nchunks) round(r * NW, r);
    } else {
      for (int base = 0; base < nchunks; base += NW) round(base, 0);
    }
    if (wave < NT * MT)
      store_out4(out, ldo, (wave % MT) * 16 + r16, (tile * NT + wave / MT) * 16 + 4 * kg, M, N, total, out_vec_ok);
  }
}

// The streaming kernel for the gate/up projection with the activation folded in:
// w holds I gate rows, then I up rows; a workgroup streams the gate tile and the
// matching up tile together and writes  out[m, n] = silu(g) * u  with g and u the
// two projections rounded to the element type first, which is what the separate
// GEMM and SwiGLU kernels compute (kernels/triton_kernels/silu_mul.py:64-87).
// M <= 16, K <= 4096 (activations resident in registers).
template <int W, int MT, int RC, int NW = SK_WAVES>
__global__ __launch_bounds__(64 * NW) void gemm_stream_swiglu_kernel(elem_t* __restrict__ out,
                                                                           const elem_t* __restrict__ act,
                                                                           const elem_t* __restrict__ w, int M, int I,
                                                                           int K, int64_t lda, int64_t ldo,
                                                                           int out_vec_ok) {
  static_assert(KC_SLABS % W == 0, "the window must divide a chunk");
  static_assert(MT * RC <= 2, "two chunk tiles of activations stay in registers: two tiles of a chunk or two chunks of a tile");
  __shared__ f32x4 part[2][RC][NW][2 * MT][64];      // two sets, used in turn: one barrier per tile

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int nchunks = K / KC;
  const int ntiles = (I + 15) / 16;

  // Wave w has chunks w, w + 8, ...: RC of them (chunks beyond K are read as the last and not used).
  frag_t wg[W], wu[W], abuf[RC * KC_SLABS][MT];
#pragma unroll
  for (int r = 0; r < RC; ++r) {
    const int c = min(r * NW + wave, nchunks - 1);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const elem_t* arow = act + (int64_t)min(mt * 16 + r16, M - 1) * lda + kg * VK_VEC;
#pragma unroll
      for (int s = 0; s < KC_SLABS; ++s)
        abuf[r * KC_SLABS + s][mt] = *reinterpret_cast<const frag_t*>(arow + c * KC + s * VK_SLAB);
    }
  }
  // Slab g of this wave's stream over a tile: chunk (g / 16) * 8 + wave, slab g % 16 of it.
  const int my_chunks = wave < nchunks ? (nchunks - wave + NW - 1) / NW : 0;     // <= RC
  const int my_slabs = my_chunks * KC_SLABS;
  auto issue = [&](int tile, int g, int slot) {
    const int64_t row = min(tile * 16 + r16, I - 1);
    const int c = (g / KC_SLABS) * NW + wave;
    const elem_t* p = w + row * K + kg * VK_VEC + (int64_t)c * KC + (g % KC_SLABS) * VK_SLAB;
    wg[slot] = *reinterpret_cast<const frag_t*>(p);
    wu[slot] = *reinterpret_cast<const frag_t*>(p + (int64_t)I * K);
  };

  int tile = blockIdx.x;
  const bool active = my_chunks > 0;
  if (tile < ntiles && active) {
#pragma unroll
    for (int i = 0; i < W; ++i) issue(tile, i, i);
  }
  int parity = 0;
  for (; tile < ntiles; tile += gridDim.x) {
    const int nt = tile + gridDim.x;
    const bool has_next = nt < ntiles;
#pragma unroll
    for (int r = 0; r < RC; ++r) {
      f32x4 ag[MT], au[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) ag[mt] = au[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (r < my_chunks) {
#pragma unroll
        for (int i = 0; i < KC_SLABS; ++i) {
          const int slot = i % W;
          const frag_t fg = wg[slot], fu = wu[slot];
          const int g = r * KC_SLABS + i + W;             // the slab that takes this slot
          if (g < my_slabs) issue(tile, g, slot);
          else if (has_next) issue(nt, g - my_slabs, slot);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            ag[mt] = mma_slab(fg, abuf[r * KC_SLABS + i][mt], ag[mt]);
            au[mt] = mma_slab(fu, abuf[r * KC_SLABS + i][mt], au[mt]);
          }
        }
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        part[parity][r][wave][2 * mt][lane] = ag[mt];
        part[parity][r][wave][2 * mt + 1][lane] = au[mt];
      }
    }
    __syncthreads();
    if (wave < MT) {       // wave mt adds up, in chunk order, and finishes the rows of activation tile mt
      f32x4 tg = {0.f, 0.f, 0.f, 0.f}, tu = {0.f, 0.f, 0.f, 0.f};
      for (int c = 0; c < nchunks; ++c) {
        const f32x4 pg = part[parity][c / NW][c % NW][2 * wave][lane];
        const f32x4 pu = part[parity][c / NW][c % NW][2 * wave + 1][lane];
        tg.x = tg.x + pg.x; tg.y = tg.y + pg.y; tg.z = tg.z + pg.z; tg.w = tg.w + pg.w;
        tu.x = tu.x + pu.x; tu.y = tu.y + pu.y; tu.z = tu.z + pu.z; tu.w = tu.w + pu.w;
      }
      const float g[4] = {round_to_elem(tg.x), round_to_elem(tg.y), round_to_elem(tg.z), round_to_elem(tg.w)};
      const float u[4] = {round_to_elem(tu.x), round_to_elem(tu.y), round_to_elem(tu.z), round_to_elem(tu.w)};
      f32x4 y;
      y.x = (g[0] * (1.0f / (1.0f + expf(-g[0])))) * u[0];
      y.y = (g[1] * (1.0f / (1.0f + expf(-g[1])))) * u[1];
      y.z = (g[2] * (1.0f / (1.0f + expf(-g[2])))) * u[2];
      y.w = (g[3] * (1.0f / (1.0f + expf(-g[3])))) * u[3];
      store_out4(out, ldo, wave * 16 + r16, tile * 16 + 4 * kg, M, I, y, out_vec_ok);
    }
    parity ^= 1;
  }
}

// ------------------------------------------------------------------- tiled
// Workgroup of four waves (2 x 2); a wave owns FN x FM tiles of 16 x 16, so the
// workgroup's tile is (32 FN) weight rows by (32 FM) activation rows.  K moves
// through LDS two slabs at a time, double-buffered; 16-byte columns of a tile
// row are XOR-swizzled by the row so that fragment reads do not collide.
#define T_ROWB 128                     // LDS bytes per tile row: two slabs
#define T_CHUNK_TILES (KC_SLABS / 2)   // K tiles (of two slabs) per chunk

template <int FN, int FM>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(elem_t* __restrict__ out, const elem_t* __restrict__ act,
                                                         const elem_t* __restrict__ w, int M, int N, int K,
                                                         int64_t lda, int64_t ldo, int out_vec_ok) {
  constexpr int BN = 32 * FN, BM = 32 * FM;
  constexpr int W_BYTES = BN * T_ROWB, A_BYTES = BM * T_ROWB, BUF_BYTES = W_BYTES + A_BYTES;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [buffer][w tile, act tile]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int wn = wave & 1, wm = wave >> 1;
  const int n_blk = blockIdx.x * BN, m_blk = blockIdx.y * BM;
  const int nslabs = (K + VK_SLAB - 1) / VK_SLAB;
  const int ntiles = (nslabs + 1) / 2;

  // Global -> LDS mapping: thread loads 16 bytes at column c16 of rows lrow + 32*i.
  const int lrow = tid >> 3, c16 = tid & 7;
  const elem_t* gw[FN];
  const elem_t* ga[FM];
  bool gw_ok[FN], ga_ok[FM];
#pragma unroll
  for (int i = 0; i < FN; ++i) {
    const int n = n_blk + lrow + 32 * i;
    gw_ok[i] = n < N;
    gw[i] = w + (int64_t)(gw_ok[i] ? n : 0) * K + c16 * VK_VEC;
  }
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int m = m_blk + lrow + 32 * i;
    ga_ok[i] = m < M;
    ga[i] = act + (int64_t)(ga_ok[i] ? m : 0) * lda + c16 * VK_VEC;
  }

  frag_t rw[FN], ra[FM];
  auto gload = [&](int kt) {
    const int k = kt * 2 * VK_SLAB;
    const bool kok = k + c16 * VK_VEC < K;
#pragma unroll
    for (int i = 0; i < FN; ++i) rw[i] = load_frag(gw[i] + k, gw_ok[i] && kok);
#pragma unroll
    for (int i = 0; i < FM; ++i) ra[i] = load_frag(ga[i] + k, ga_ok[i] && kok);
  };
  auto lstore = [&](int buf) {
    unsigned char* base = lds + buf * BUF_BYTES;
    const int col = (c16 ^ (lrow & 7)) * 16;
#pragma unroll
    for (int i = 0; i < FN; ++i) *reinterpret_cast<frag_t*>(base + (lrow + 32 * i) * T_ROWB + col) = rw[i];
#pragma unroll
    for (int i = 0; i < FM; ++i) *reinterpret_cast<frag_t*>(base + W_BYTES + (lrow + 32 * i) * T_ROWB + col) = ra[i];
  };

  f32x4 acc[FN][FM], total[FN][FM];
#pragma unroll
  for (int i = 0; i < FN; ++i)
#pragma unroll
    for (int j = 0; j < FM; ++j) {
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      total[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

  gload(0);
  lstore(0);
  __syncthreads();

  for (int kt = 0; kt < ntiles; ++kt) {
    const unsigned char* base = lds + (kt & 1) * BUF_BYTES;
    if (kt + 1 < ntiles) gload(kt + 1);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      frag_t wf[FN], af[FM];
      const int col = ((s * 4 + kg) ^ (r16 & 7)) * 16;
#pragma unroll
      for (int i = 0; i < FN; ++i)
        wf[i] = *reinterpret_cast<const frag_t*>(base + (wn * 16 * FN + i * 16 + r16) * T_ROWB + col);
#pragma unroll
      for (int j = 0; j < FM; ++j)
        af[j] = *reinterpret_cast<const frag_t*>(base + W_BYTES + (wm * 16 * FM + j * 16 + r16) * T_ROWB + col);
#pragma unroll
      for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j) acc[i][j] = mma_slab(wf[i], af[j], acc[i][j]);
    }
    if ((kt + 1) % T_CHUNK_TILES == 0 || kt + 1 == ntiles) {
#pragma unroll
      for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j) {
          total[i][j].x = total[i][j].x + acc[i][j].x;
          total[i][j].y = total[i][j].y + acc[i][j].y;
          total[i][j].z = total[i][j].z + acc[i][j].z;
          total[i][j].w = total[i][j].w + acc[i][j].w;
          acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    if (kt + 1 < ntiles) lstore((kt & 1) ^ 1);
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < FN; ++i)
#pragma unroll
    for (int j = 0; j < FM; ++j)
      store_out4(out, ldo, m_blk + wm * 16 * FM + j * 16 + r16, n_blk + wn * 16 * FN + i * 16 + 4 * kg, M, N,
                 total[i][j], out_vec_ok);
}

template <int FN, int FM>
static int launch_tiled(elem_t* out, const elem_t* act, const elem_t* w, int M, int N, int K, int64_t lda, int64_t ldo,
                        int vec_ok, hipStream_t st) {
  constexpr int BN = 32 * FN, BM = 32 * FM;
  const size_t smem = 2 * (size_t)(BN + BM) * T_ROWB;
  static bool configured = false;
  if (!configured) {
    if (smem > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)gemm_tiled_kernel<FN, FM>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)smem);
    configured = true;
  }
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  VK_REQUIRE(grid.y <= 65535, "gemm: too many rows (%d)", M);
  gemm_tiled_kernel<FN, FM><<<grid, 256, smem, st>>>(out, act, w, M, N, K, lda, ldo, vec_ok);
  return vk_check_launch("gemm_tiled");
}

// --------------------------------------------------------------- pipelined
// The tiled kernel for K a multiple of 64 bytes-per-row tiles (two slabs), with
// what the other lacks to keep the MFMA units fed: tiles go from global memory
// straight into LDS (global_load_lds_dwordx4, no registers in between) and S
// stages are in flight, so a tile's latency is hidden behind the S-1 tiles
// computed meanwhile.  One barrier per K tile.  Rows beyond N or M are clamped
// (their results are dropped).  Same tile shape, swizzle and reduction order as
// gemm_tiled_kernel<4, 4>.
__device__ __forceinline__ void wait_vmcnt(int n) {
  // s_waitcnt with only vmcnt set: vmcnt is bits [3:0] and [15:14]; expcnt and lgkmcnt left at their maxima.
  switch (n) {
    case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
    case 8: __builtin_amdgcn_s_waitcnt(0x0F78); break;
    case 16: __builtin_amdgcn_s_waitcnt(0x4F70); break;
    case 24: __builtin_amdgcn_s_waitcnt(0x4F78); break;
    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
  }
}

// With SWIGLU the weight holds N gate rows, then N up rows, and the output has N columns: a workgroup
// takes 64 gate rows and the matching 64 up rows as its 128 weight rows (the waves with wn = 0 the
// gate, those with wn = 1 the up projection), and at the end the up values pass through LDS to the
// waves that hold the gate values, which write  silu(g) * u  with g and u rounded to the element type
// first: the bits of the plain projection followed by swiglu_kernel.
// 16 bytes per lane from global memory into LDS at dst + 16 * lane.  In a function of its own: called
// with template-dependent arguments from inside the kernel template, the builtin keeps the compiler
// from emitting the kernel's host-side stub.
__device__ __forceinline__ void pipe_load_to_lds16(const elem_t* src, unsigned char* dst) {
  __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
}

// The same load with its address in two parts: a base held in scalar registers, the same for every lane, and a
// 32-bit offset per lane.  The compiler's own form of it adds base and offset in vector registers before every
// load (it moves what does not change along K out of the loop and is left with a vector sum); written out, the
// advancing base costs two scalar additions per K tile for all loads together.  lds_addr: the wave's 1 KB
// block in LDS, below 64 KB.
__device__ __forceinline__ void pipe_load_to_lds16_sv(const unsigned char* sbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(sbase), "s"(lds_addr) : "memory");     // m0 is the compiler's scratch: it sets it anew before every use of its own
}
__device__ __forceinline__ unsigned lds_offset_of(const unsigned char* p) {
  return (unsigned)(unsigned long)((__attribute__((address_space(3))) const void*)p);
}

// FNW: 16-row weight fragments per wave, 2 to 5: a workgroup takes 32 FNW weight rows.  4 is the square tile; 2
// gives twice the workgroups, for grids that would leave compute units with one workgroup or none; 3 and 5 are
// for grids whose last round of workgroups would otherwise run nearly empty (pipe_fragments_by_rounds).  Six
// would need more than the 256 registers of a wave.
// One 4-byte load per lane whose value nobody reads: it brings the lane's 128-byte line into the second-level
// cache ahead of the LDS-direct load that will want it.  `keep` is one register that every such load writes
// (in order, so they may overlap) and that stays allocated to the end of the kernel.
__device__ __forceinline__ void pipe_touch_line(const unsigned char* sbase, unsigned voff, unsigned& keep) {
  asm volatile("global_load_dword %0, %1, %2 sc1" : "+v"(keep) : "v"(voff), "s"(sbase) : "memory");
}
template <int N_>
__device__ __forceinline__ void wait_vmcnt_n() {             // vmcnt(N_), N_ below 64; the other counters at their maxima
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N_ & 0xF) | ((N_ >> 4) << 14));
}

// PFD > 0: every wave touches, PFD tiles ahead, the 64 rows of the workgroup's tiles that are its share.
template <int S, bool WHOLE, bool SWIGLU, int FNW = 4, int PFD = 0>
__global__ __launch_bounds__(256, 2) void gemm_pipe_kernel(elem_t* __restrict__ out, const elem_t* __restrict__ act,
                                                        const elem_t* __restrict__ w, int M, int N, int K,
                                                        int64_t lda, int64_t ldo, int out_vec_ok, int band_w) {
  static_assert(FNW >= 2 && FNW <= 5 && (FNW == 4 || !SWIGLU), "two to five weight fragments per wave; four with SwiGLU");
  static_assert(PFD == 0 || FNW == 2 || FNW == 4, "the touch-ahead wants a wave's 64 rows to be of one kind");
  constexpr int BN = 32 * FNW;                          // weight rows of the workgroup
  constexpr int W_BYTES = BN * T_ROWB, STAGE_BYTES = W_BYTES + 128 * T_ROWB;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [stage][w tile, act tile]

  // The wave number as a scalar: what depends on it alone (LDS addresses, which rows a load brings)
  // then needs no vector registers.
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kg = lane >> 4;
  const int wn = wave & 1, wm = wave >> 1;
  // Workgroups start in the order of their linear index.  That order walks bands of band_w column
  // blocks: all row blocks of a band before the next band, so that a band's weights are read from HBM
  // once and found in the caches by the other row blocks (a matrix larger than the memory-side cache
  // would otherwise be streamed once per row block).
  int nb = blockIdx.x, mb = blockIdx.y;
  if (band_w < (int)gridDim.x) {
    const int lin = blockIdx.y * gridDim.x + blockIdx.x;
    const int per_band = band_w * gridDim.y;
    const int band = lin / per_band, r = lin - band * per_band;
    const int w_here = min(band_w, (int)gridDim.x - band * band_w);
    mb = r / w_here;
    nb = band * band_w + (r - mb * w_here);
  }
  const int n_blk = nb * (SWIGLU ? 64 : BN), m_blk = mb * 128;
  const int ntiles = K / (2 * VK_SLAB);

  // A wave-level load moves 8 rows x 128 bytes; lane i fills LDS slot i of the 1 KB block, which is
  // row i/8, physical 16-byte column i%8, i.e. logical column (i%8) ^ (i/8).
  const int lr = lane >> 3, lc = (lane & 7) ^ lr;
  // A load's address is a base that is the same for the whole workgroup (the first weight row of the
  // block, or of its up rows; the first activation row), which advances along K as a scalar, plus a
  // 32-bit offset per lane that never changes: no vector arithmetic per load.
  const unsigned char* wbase = reinterpret_cast<const unsigned char*>(w + (int64_t)min(n_blk, N - 1) * K);
  const unsigned char* ubase = reinterpret_cast<const unsigned char*>(w + (int64_t)(N + min(n_blk, N - 1)) * K);   // SWIGLU: the up rows
  const unsigned char* abase = reinterpret_cast<const unsigned char*>(act + (int64_t)min(m_blk, M - 1) * lda);
  unsigned offw[FNW], offa[4];
#pragma unroll
  for (int j = 0; j < FNW; ++j) {
    const int row = (wave * FNW + j) * 8 + lr;
    const int local = SWIGLU ? (row < 64 ? row : row - 64) : row;                 // row of the block, gate or up
    const int clamped = min(n_blk + local, N - 1) - min(n_blk, N - 1);
    offw[j] = (unsigned)(((int64_t)clamped * K + lc * VK_VEC) * (int64_t)sizeof(elem_t));
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int clamped = min(m_blk + (wave * 4 + j) * 8 + lr, M - 1) - min(m_blk, M - 1);
    offa[j] = (unsigned)(((int64_t)clamped * lda + lc * VK_VEC) * (int64_t)sizeof(elem_t));
  }
  const unsigned lds0 = lds_offset_of(lds);
  auto issue = [&](int kt) {                 // FNW + 4 loads per wave
    const unsigned base = lds0 + (kt % S) * STAGE_BYTES;
    const int64_t kb = (int64_t)kt * 2 * VK_SLAB * (int64_t)sizeof(elem_t);
#pragma unroll
    for (int j = 0; j < FNW; ++j) {
      const bool up = SWIGLU && (wave * FNW + j) * 8 >= 64;       // a scalar: all eight rows of a load are of one kind
      pipe_load_to_lds16_sv((up ? ubase : wbase) + kb, offw[j], base + (wave * FNW + j) * 8 * T_ROWB);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) pipe_load_to_lds16_sv(abase + kb, offa[j], base + W_BYTES + (wave * 4 + j) * 8 * T_ROWB);
  };

  // The lines a wave touches ahead: row wave * 64 + lane of the workgroup's weight rows followed by its
  // activation rows (a wave's 64 rows are all weights, all up rows, or all activations).
  static_assert(PFD == 0 || S == 2, "the touch-ahead counts its loads for two stages");
  unsigned pf_off = 0, pf_keep = 0;
  const unsigned char* pf_base = wbase;
  if (PFD > 0) {
    const int r = wave * 64 + lane;
    if (wave * 64 < BN) {
      const bool up = SWIGLU && wave * 64 >= 64;
      const int local = up ? r - 64 : r;
      pf_base = up ? ubase : wbase;
      pf_off = (unsigned)((int64_t)(min(n_blk + local, N - 1) - min(n_blk, N - 1)) * K * (int64_t)sizeof(elem_t));
    } else {
      pf_base = abase;
      pf_off = (unsigned)((int64_t)(min(m_blk + min(r - BN, 127), M - 1) - min(m_blk, M - 1)) * lda * (int64_t)sizeof(elem_t));
    }
  }

  f32x4 acc[FNW][4], total[FNW][4];
#pragma unroll
  for (int i = 0; i < FNW; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      total[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

#pragma unroll
  for (int p = 0; p < S - 1; ++p)
    if (p < ntiles) issue(p);

  auto step = [&](int kt) {
    // Tile kt has landed once at most the loads of the tiles after it are outstanding (FNW + 4 per tile and wave).
    if (PFD > 0) {
      if (kt == 0) wait_vmcnt_n<0>(); else wait_vmcnt_n<1>();      // the one touch that was issued behind tile kt's loads may still fly
    } else {
      const int later = min(S - 2, ntiles - 1 - kt);
      wait_vmcnt((FNW + 4) * later);
    }
    __syncthreads();       // every wave's part of tile kt is there; everyone is done with tile kt-1's buffer
    if (kt + S - 1 < ntiles) issue(kt + S - 1);
    if (PFD > 0)           // always one, so that the count above holds: beyond the end the last tile again
      pipe_touch_line(pf_base + (int64_t)min(kt + PFD, ntiles - 1) * 2 * VK_SLAB * (int64_t)sizeof(elem_t), pf_off, pf_keep);
    const unsigned char* base = lds + (kt % S) * STAGE_BYTES;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      frag_t wf[FNW], af[4];
      const int col = ((s * 4 + kg) ^ (r16 & 7)) * 16;
#pragma unroll
      for (int i = 0; i < FNW; ++i) wf[i] = *reinterpret_cast<const frag_t*>(base + (wn * 16 * FNW + i * 16 + r16) * T_ROWB + col);
#pragma unroll
      for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const frag_t*>(base + W_BYTES + (wm * 64 + i * 16 + r16) * T_ROWB + col);
#pragma unroll
      for (int i = 0; i < FNW; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mma_slab(wf[i], af[j], acc[i][j]);
    }
#ifdef VK_BF16
    // Order for the scheduler: the first slab's reads, then the second slab's reads one by one between
    // the first slab's MFMAs, so that they return while the matrix unit works.
    constexpr int BETWEEN = FNW >= 4 ? 2 : 1;                    // MFMAs between two of the second slab's reads
    __builtin_amdgcn_sched_group_barrier(0x100, FNW + 4, 0);     // the first slab's LDS reads
#pragma unroll
    for (int q = 0; q < FNW + 4; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, BETWEEN, 0);            // MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                  // 1 LDS read
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 8 * FNW - (FNW + 4) * BETWEEN, 0);   // the first slab's other MFMAs and the second slab's
#endif
  };
  auto close_chunk = [&]() {
#pragma unroll
    for (int i = 0; i < FNW; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        total[i][j].x = total[i][j].x + acc[i][j].x;
        total[i][j].y = total[i][j].y + acc[i][j].y;
        total[i][j].z = total[i][j].z + acc[i][j].z;
        total[i][j].w = total[i][j].w + acc[i][j].w;
        acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
  };
  if (WHOLE) {
    // K is whole chunks: the tiles of a chunk are written out one after the other, so that the chunk
    // sums are touched between chunks only and need not move between register files in every tile.
    for (int kt0 = 0; kt0 < ntiles; kt0 += T_CHUNK_TILES) {
#pragma unroll
      for (int u = 0; u < T_CHUNK_TILES; ++u) step(kt0 + u);
      close_chunk();
    }
  } else {
    for (int kt = 0; kt < ntiles; ++kt) {
      step(kt);
      if ((kt + 1) % T_CHUNK_TILES == 0 || kt + 1 == ntiles) close_chunk();
    }
  }

  if (PFD > 0) {
    wait_vmcnt_n<0>();                                        // the last touches
    asm volatile("" : : "v"(pf_keep));                        // the register was theirs until here
  }
  if constexpr (SWIGLU) {
    // The two waves of a row block split the 64 output columns: the gate wave keeps columns 0..31 and
    // gets their up values, the up wave keeps columns 32..63 and gets their gate values.
    __syncthreads();            // the last tile has been read: LDS is free
    // [128 rows][16 groups of 4 columns]; a row's group g lies at place g ^ (row % 16), so that the 16 rows a
    // wave touches at once (256 bytes apart: the same banks) spread over all banks.
    f32x4* ex = reinterpret_cast<f32x4*>(lds);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f32x4& v = total[i][j];
        v.x = round_to_elem(v.x); v.y = round_to_elem(v.y); v.z = round_to_elem(v.z); v.w = round_to_elem(v.w);
        if ((i < 2) == (wn == 1)) ex[(wm * 64 + j * 16 + r16) * 16 + ((i * 4 + kg) ^ r16)] = v;    // what the other wave needs
      }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if ((i < 2) != (wn == 0)) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 o = ex[(wm * 64 + j * 16 + r16) * 16 + ((i * 4 + kg) ^ r16)];
        const f32x4 g = wn == 0 ? total[i][j] : o, u = wn == 0 ? o : total[i][j];
        f32x4 y;
        y.x = (g.x * (1.0f / (1.0f + expf(-g.x)))) * u.x;
        y.y = (g.y * (1.0f / (1.0f + expf(-g.y)))) * u.y;
        y.z = (g.z * (1.0f / (1.0f + expf(-g.z)))) * u.z;
        y.w = (g.w * (1.0f / (1.0f + expf(-g.w)))) * u.w;
        store_out4(out, ldo, m_blk + wm * 64 + j * 16 + r16, n_blk + i * 16 + 4 * kg, M, N, y, out_vec_ok);
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < FNW; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      store_out4(out, ldo, m_blk + wm * 64 + j * 16 + r16, n_blk + wn * 16 * FNW + i * 16 + 4 * kg, M, N, total[i][j],
                 out_vec_ok);
}

// Column blocks of a band in the tile kernel (0: no bands).  64: the 512 workgroups that run at a time
// then are 8 row blocks of 64 column blocks, and the 64 of them on a chip part (workgroup i runs on part
// i % 8) are 8 row blocks of 8 column blocks: the fewest distinct tiles for its cache.  Measured on
// MI355X, gate/up with SwiGLU at 2,048 to 8,192 rows: 12,288 x 4,096 weights 950 -> 1,090 TFLOP/s,
// 25,600 x 5,120 (524 MB, more than the memory-side cache holds) 600 -> 1,040; 51 or 76 column blocks,
// which move a column block from part to part, 780 to 830.
static const int pipe_band_blocks = 64;

template <int S, bool SWIGLU = false, int FNW = 4>
static int launch_pipe(elem_t* out, const elem_t* act, const elem_t* w, int M, int N, int K, int64_t lda, int64_t ldo,
                       int vec_ok, hipStream_t st) {
  constexpr int BN = SWIGLU ? 64 : 32 * FNW;                         // output columns of a workgroup
  const size_t smem = (size_t)S * (32 * FNW + 128) * T_ROWB;         // also holds the 32 KB that SWIGLU passes between waves
  static bool configured = false;
  if (!configured) {
    (void)hipFuncSetAttribute((const void*)gemm_pipe_kernel<S, true, SWIGLU, FNW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    (void)hipFuncSetAttribute((const void*)gemm_pipe_kernel<S, false, SWIGLU, FNW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    configured = true;
  }
  dim3 grid((N + BN - 1) / BN, (M + 127) / 128);
  VK_REQUIRE(grid.y <= 65535, "gemm: too many rows (%d)", M);
  const int band_w = (pipe_band_blocks > 0 && grid.y > 1 && (int)grid.x > pipe_band_blocks) ? pipe_band_blocks : (int)grid.x;
  if constexpr (S == 2 && (FNW == 2 || FNW == 4)) {
    // No more workgroups than compute units: each waits for its own loads with nothing to run meanwhile, and
    // touching the lines four tiles ahead brings them into the second-level cache in time (300 rows, 4,096 x
    // 12,288: 146 -> 112 us).  With more workgroups the touches cost more than they bring: the path from
    // that cache into LDS is as busy as the MFMA unit (2,048 rows: 1,057 -> 660 TFLOP/s).
    if (K % KC == 0 && (int64_t)grid.x * grid.y <= device_cus()) {
      static bool touched = false;
      if (!touched) {
        (void)hipFuncSetAttribute((const void*)gemm_pipe_kernel<S, true, SWIGLU, FNW, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        touched = true;
      }
      gemm_pipe_kernel<S, true, SWIGLU, FNW, 4><<<grid, 256, smem, st>>>(out, act, w, M, N, K, lda, ldo, vec_ok, band_w);
      return vk_check_launch("gemm_pipe");
    }
  }
  if (K % KC == 0) gemm_pipe_kernel<S, true, SWIGLU, FNW><<<grid, 256, smem, st>>>(out, act, w, M, N, K, lda, ldo, vec_ok, band_w);
  else gemm_pipe_kernel<S, false, SWIGLU, FNW><<<grid, 256, smem, st>>>(out, act, w, M, N, K, lda, ldo, vec_ok, band_w);
  return vk_check_launch("gemm_pipe");
}

// ------------------------------------------------------------------ mid
// 17 to 64 rows.  The streaming kernels read all activations once per 16 weight rows, which at 64 rows
// is four times the weights and binds them to the second-level cache.  Here a workgroup of eight waves
// takes 64 weight rows: wave (nt, kh) streams weight tile nt (16 rows) for the chunks kh, kh + 2, ...
// into registers with a rolling window, as the streaming kernels do, and the activations of the two
// chunks in work go into LDS once for all waves (global_load_lds, a quarter chunk at a time, two
// buffers).  After a pair of chunks the waves with kh = 1 hand their chunk sum over through LDS and the
// waves with kh = 0 add both to the total, in chunk order.  K is a multiple of 512.
//
// Waits: the barrier of a step is a bare s_barrier (a __syncthreads would wait for every weight load in
// flight); a wave waits for its part of the activation loads by count: they are followed by exactly
// MID_QS weight loads before the next step begins (MID_W at the start), kept so by scheduling barriers.
#define MID_QS 4                       // slabs per step
#define MID_W 8                        // weight slabs in flight per wave
__device__ __forceinline__ void mid_wait_vmcnt_4() { __builtin_amdgcn_s_waitcnt(0x0F74); }
__device__ __forceinline__ void mid_wait_vmcnt_w() { static_assert(MID_W == 8, "vmcnt(8)"); __builtin_amdgcn_s_waitcnt(0x0F78); }
__device__ __forceinline__ void mid_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ void mid_load_to_lds16(const elem_t* src, unsigned char* dst) {
  __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
}

// SWIGLU (one chunk in work, KH = 1): w holds N gate rows, then N up rows; waves 0..GT-1 take GT gate
// tiles, waves GT..2GT-1 the matching up tiles, and out[m, n] = silu(g) * u with g and u rounded to the
// element type first, as the separate kernels compute it.  With GT < 4 the other waves only help to bring
// in the activations: 12288 gate rows are 256 workgroups of three tiles, one for every compute unit,
// where four tiles a workgroup leave a quarter of them idle.
template <int MT, int KH, bool SWIGLU = false, int GT = 4>
__global__ __launch_bounds__(512) void gemm_mid_kernel(elem_t* __restrict__ out, const elem_t* __restrict__ act,
                                                       const elem_t* __restrict__ w, int M, int N, int K,
                                                       int64_t lda, int64_t ldo, int out_vec_ok) {
  static_assert(!SWIGLU || KH == 1, "the SwiGLU epilogue pairs the waves of one chunk");
  static_assert(GT == 4 || (SWIGLU && GT >= 2 && GT < 4), "fewer gate tiles only with the SwiGLU epilogue");
  constexpr int NTW = 8 / KH;                       // waves side by side along the weight rows
  constexpr int ACTIVE = SWIGLU ? 2 * GT : 8;       // waves that stream weights
  constexpr int STEPS = KC_SLABS / MID_QS;          // steps per chunk
  constexpr int ROW_B = MID_QS * 64;                // bytes of an activation row in a step: 256
  constexpr int HALF_B = 16 * MT * ROW_B;           // one chunk's part of a buffer
  constexpr int BUF_B = KH * HALF_B;
  constexpr int DMA = MT * KH / 2;                  // activation loads per wave and step (8 KH MT / 2 in all... 4 rows each)
  static_assert((MT * KH) % 2 == 0, "the activation loads divide evenly over the waves");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [2 buffers][kh][16 MT rows][256 B], then part
  f32x4* part = reinterpret_cast<f32x4*>(lds + 2 * BUF_B);              // [KH - 1][NTW tiles][MT][64 lanes]

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, kg = lane >> 4;
  const int nt = wave % NTW, kh = wave / NTW;
  const bool active = ACTIVE == 8 || wave < ACTIVE;
  const int row0 = blockIdx.y * 16 * MT;            // more than 16 MT rows: one block of them per blockIdx.y
  const int nchunks = K / KC, ngroups = (nchunks + KH - 1) / KH;     // group: KH chunks in work together
  const int nsteps = ngroups * STEPS;
  const int last_full = nchunks - (ngroups - 1) * KH;                // chunks of the last group: 1 .. KH

  // Weights: row of this wave's tile, chunk sequence kh, kh + KH, ...; a chunk beyond the last is read as
  // the last (and not used), so that every wave issues the same number of loads.
  const int out_col0 = SWIGLU ? (int)blockIdx.x * 16 * GT + (nt % GT) * 16 : (int)blockIdx.x * 16 * NTW + nt * 16;
  const int64_t wrow_i = SWIGLU ? (int64_t)min(nt / GT, 1) * N + min(out_col0 + r16, N - 1) : min(out_col0 + r16, N - 1);
  const elem_t* wrow = w + wrow_i * K + kg * VK_VEC;
  frag_t wbuf[MID_W];
  auto issue_w = [&](int g, int slot) {              // g: this wave's slab number; slot = g % MID_W
    const int gg = min(g, nsteps * MID_QS - 1);
    const int c = min(KH * (gg / KC_SLABS) + kh, nchunks - 1);
    wbuf[slot] = *reinterpret_cast<const frag_t*>(wrow + (int64_t)c * KC + (gg % KC_SLABS) * VK_SLAB);
  };
  // Activations of a step: KH * 16 MT rows of 256 bytes; a wave-level load fills 4 rows, lane i the
  // 16-byte column i % 16 of row i / 16, which holds the logical column (i % 16) ^ (row % 16).
  const elem_t* asrc[DMA];
  int adst[DMA], ah[DMA];
#pragma unroll
  for (int j = 0; j < DMA; ++j) {
    const int id = wave * DMA + j;                   // 0 .. 4 MT KH - 1
    const int h = id / (4 * MT), row = (id % (4 * MT)) * 4 + (lane >> 4);
    ah[j] = h;
    asrc[j] = act + (int64_t)min(row0 + row, M - 1) * lda + (((lane & 15) ^ (row & 15)) * VK_VEC);
    adst[j] = h * HALF_B + (id % (4 * MT)) * 4 * ROW_B;
  }
  auto issue_a = [&](int t) {                        // step t of the workgroup
    const int tt = min(t, nsteps - 1);
    const int group = tt / STEPS, q = tt % STEPS;
    unsigned char* base = lds + (t & 1) * BUF_B;
#pragma unroll
    for (int j = 0; j < DMA; ++j) {
      const int c = min(group * KH + ah[j], nchunks - 1);    // beyond the last chunk: the last again (not used)
      mid_load_to_lds16(asrc[j] + (int64_t)c * KC + q * MID_QS * VK_SLAB, base + adst[j]);
    }
  };

  f32x4 acc[MT], total[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = total[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  // The chunk sums of a complete group join the total in chunk order: this wave's own, then the others'.
  auto close_group = [&](int chunks_in_group) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      total[mt].x = total[mt].x + acc[mt].x; total[mt].y = total[mt].y + acc[mt].y;
      total[mt].z = total[mt].z + acc[mt].z; total[mt].w = total[mt].w + acc[mt].w;
#pragma unroll
      for (int h = 1; h < KH; ++h) {
        if (h < chunks_in_group) {
          const f32x4 p = part[(((h - 1) * NTW + nt) * MT + mt) * 64 + lane];
          total[mt].x = total[mt].x + p.x; total[mt].y = total[mt].y + p.y;
          total[mt].z = total[mt].z + p.z; total[mt].w = total[mt].w + p.w;
        }
      }
    }
  };

  constexpr int TURN = MID_W / MID_QS;      // steps in one turn of the weight window
  static_assert(STEPS % TURN == 0, "a turn of the weight window is a whole number of steps");
  issue_a(0);
  __builtin_amdgcn_sched_barrier(0);
  if (active) {
#pragma unroll
    for (int i = 0; i < MID_W; ++i) issue_w(i, i);
    __builtin_amdgcn_sched_barrier(0);
    for (int t2 = 0; t2 < nsteps; t2 += TURN) {
#pragma unroll
      for (int u = 0; u < TURN; ++u) {         // written out: the window's slots are then fixed registers
        const int t = t2 + u;
        if (t == 0) mid_wait_vmcnt_w(); else mid_wait_vmcnt_4();
        mid_barrier();          // step t's activations are in LDS; everyone is done with the other buffer
        const int group = t / STEPS, q = t % STEPS;
        if (q == 0 && group > 0) {
          if (kh == 0) close_group(KH);           // the group before is complete
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        __builtin_amdgcn_sched_barrier(0);
        issue_a(t + 1);
        __builtin_amdgcn_sched_barrier(0);
        const unsigned char* abase = lds + (t & 1) * BUF_B + kh * HALF_B;
#pragma unroll
        for (int s = 0; s < MID_QS; ++s) {
          const int g = t * MID_QS + s;
          const frag_t fw = wbuf[u * MID_QS + s];
          frag_t fa[MT];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            fa[mt] = *reinterpret_cast<const frag_t*>(abase + (mt * 16 + r16) * ROW_B + (((s * 4 + kg) ^ r16) << 4));
          issue_w(g + MID_W, u * MID_QS + s);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[mt] = mma_slab(fw, fa[mt], acc[mt]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (q == STEPS - 1 && kh > 0) {
          // This wave's chunk of the group is complete: hand it over (one beyond the last chunk is not used).
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) part[(((kh - 1) * NTW + nt) * MT + mt) * 64 + lane] = acc[mt];
        }
      }
    }
  } else {
    // A wave without weights only brings in its share of the activations: the same barriers, and nothing
    // in flight but those loads.
    for (int t = 0; t < nsteps; ++t) {
      __builtin_amdgcn_s_waitcnt(0x0F70);
      mid_barrier();
      issue_a(t + 1);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);      // the loads issued beyond the end
  mid_barrier();
  if (kh == 0) {
    close_group(last_full);
    if (SWIGLU) {
      // Every wave is past the barrier above, so the activation buffers are free: the up waves leave
      // their sums there for the gate waves of the same columns.
      f32x4* ex = reinterpret_cast<f32x4*>(lds);       // [GT tiles][MT][64 lanes]
      if (nt >= GT && active) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) ex[((nt - GT) * MT + mt) * 64 + lane] = total[mt];
      }
      __syncthreads();
      if (nt < GT) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const f32x4 t = total[mt], o = ex[(nt * MT + mt) * 64 + lane];
          const float g[4] = {round_to_elem(t.x), round_to_elem(t.y), round_to_elem(t.z), round_to_elem(t.w)};
          const float u[4] = {round_to_elem(o.x), round_to_elem(o.y), round_to_elem(o.z), round_to_elem(o.w)};
          f32x4 y;
          y.x = (g[0] * (1.0f / (1.0f + expf(-g[0])))) * u[0];
          y.y = (g[1] * (1.0f / (1.0f + expf(-g[1])))) * u[1];
          y.z = (g[2] * (1.0f / (1.0f + expf(-g[2])))) * u[2];
          y.w = (g[3] * (1.0f / (1.0f + expf(-g[3])))) * u[3];
          store_out4(out, ldo, row0 + mt * 16 + r16, out_col0 + 4 * kg, M, N, y, out_vec_ok);
        }
      }
      return;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      store_out4(out, ldo, row0 + mt * 16 + r16, out_col0 + 4 * kg, M, N, total[mt], out_vec_ok);
  }
}

// N: weight rows, or with SWIGLU the gate rows (and as many up rows after them).
template <int MT, int KH, bool SWIGLU = false, int GT = 4>
static int launch_mid(elem_t* out, const elem_t* act, const elem_t* w, int M, int N, int K, int64_t lda, int64_t ldo,
                      int vec_ok, hipStream_t st) {
  constexpr int NTW = 8 / KH;
  constexpr int COLS = SWIGLU ? 16 * GT : 16 * NTW; // output columns of a workgroup
  const size_t smem = (size_t)2 * KH * 16 * MT * (MID_QS * 64) + (size_t)(KH - 1) * NTW * MT * 64 * sizeof(f32x4);
  static_assert(!SWIGLU || 2 * 16 * MT * (MID_QS * 64) >= 4 * MT * 64 * (int)sizeof(f32x4), "the exchange fits the activation buffers");
  static bool configured = false;
  if (!configured) {
    (void)hipFuncSetAttribute((const void*)gemm_mid_kernel<MT, KH, SWIGLU, GT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    configured = true;
  }
  // Blocks of 16 MT rows side by side: those of a weight tile run at about the same time, and on the same
  // chip part when the grid's width is a multiple of eight, so that all but one find it in its cache.
  const dim3 grid((N + COLS - 1) / COLS, (M + 16 * MT - 1) / (16 * MT));
  gemm_mid_kernel<MT, KH, SWIGLU, GT><<<grid, 512, smem, st>>>(out, act, w, M, N, K, lda, ldo, vec_ok);
  return vk_check_launch("gemm_mid");
}

// ---------------------------------------------------------------- split
// 17 to 64 rows and few weight rows: the kernels above give such a product a workgroup or less per compute
// unit, each walking a long stretch of K on its own with a window of loads that one latency drains.  Here
// a workgroup takes 16 NTW weight rows of ONE chunk: a wave's 16 rows x 512 elements are all in flight at
// once, the chunk of the activations goes into LDS once for its waves, and the chunk sums go to a
// workspace [chunk][weight tile][activation tile][lane]; a second kernel adds them in chunk order to a
// zero total, which is what every other kernel computes, and writes the output (with SWIGLU: of
// silu(g) * u, g and u rounded to the element type first).  16-bit elements only.
#ifdef VK_BF16
template <int MT, int NTW>
__global__ __launch_bounds__(64 * NTW) void gemm_split_kernel(f32x4* __restrict__ partial, const elem_t* __restrict__ act,
                                                              const elem_t* __restrict__ w, int M, int N, int K,
                                                              int64_t lda, int ntiles16) {
  constexpr int ROW_B = KC * (int)sizeof(elem_t);           // bytes of an activation row of a chunk: 1024
  static_assert(ROW_B == 64 * 16, "a wave-level load fills one activation row");
  __shared__ __attribute__((aligned(16))) unsigned char lds[16 * MT * ROW_B];

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, kg = lane >> 4;
  const int c = blockIdx.y;
  const int tile = blockIdx.x * NTW + wave;                  // 16-row weight tile; beyond the last: clamped rows, nothing stored

  // Activations first: row r of the chunk lies at lds + r * 1024, its logical 16-byte column j at physical
  // column j ^ (r % 16); lane i of a wave-level load fills physical column i.
#pragma unroll
  for (int j = 0; j < 16 * MT / NTW; ++j) {
    const int r = wave + j * NTW;
    __builtin_amdgcn_global_load_lds(act + (int64_t)min(r, M - 1) * lda + (int64_t)c * KC + ((lane ^ (r & 15)) * VK_VEC),
                                     (__attribute__((address_space(3))) void*)(lds + r * ROW_B), 16, 0, 0);
  }
  __builtin_amdgcn_sched_barrier(0);
  const elem_t* wrow = w + (int64_t)min(tile * 16 + r16, N - 1) * K + (int64_t)c * KC + kg * VK_VEC;
  frag_t wbuf[KC_SLABS];
#pragma unroll
  for (int s = 0; s < KC_SLABS; ++s) wbuf[s] = *reinterpret_cast<const frag_t*>(wrow + s * VK_SLAB);
  __builtin_amdgcn_sched_barrier(0);
  static_assert(KC_SLABS == 16, "vmcnt(16) below: the weight loads are the 16 issued last");
  __builtin_amdgcn_s_waitcnt(0x4F70);      // vmcnt(16): this wave's activation rows are in LDS; its weights still fly
  __syncthreads();

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < KC_SLABS; ++s) {
    frag_t fa[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      fa[mt] = *reinterpret_cast<const frag_t*>(lds + (mt * 16 + r16) * ROW_B + (((s * 4 + kg) ^ r16) << 4));
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = mma_slab(wbuf[s], fa[mt], acc[mt]);
  }
  if (tile < ntiles16) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) partial[(((int64_t)c * ntiles16 + tile) * MT + mt) * 64 + lane] = acc[mt];
  }
}

// One thread per (weight tile, activation tile, lane): the chunk sums in chunk order.  up_tiles > 0: the
// tile and the one up_tiles after it are the gate and the up projection of the same output columns.
template <int MT>
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(elem_t* __restrict__ out, const f32x4* __restrict__ partial,
                                                                int M, int N, int64_t ldo, int nchunks, int ntiles16,
                                                                int up_tiles, int out_vec_ok) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int lane = (int)(t & 63), mt = (int)((t >> 6) % MT);
  const int tile = (int)(t / (64 * MT));
  const int out_tiles = up_tiles > 0 ? up_tiles : ntiles16;
  if (tile >= out_tiles) return;
  const int r16 = lane & 15, kg = lane >> 4;
  auto sum = [&](int tl) {
    f32x4 total = {0.f, 0.f, 0.f, 0.f};
    const f32x4* p0 = partial + ((int64_t)tl * MT + mt) * 64 + lane;
    const int64_t stride = (int64_t)ntiles16 * MT * 64;
    int c = 0;
    for (; c + 8 <= nchunks; c += 8) {         // eight loads in flight, added in chunk order
      f32x4 p[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = p0[(c + i) * stride];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        total.x = total.x + p[i].x; total.y = total.y + p[i].y; total.z = total.z + p[i].z; total.w = total.w + p[i].w;
      }
    }
    for (; c < nchunks; ++c) {
      const f32x4 p = p0[c * stride];
      total.x = total.x + p.x; total.y = total.y + p.y; total.z = total.z + p.z; total.w = total.w + p.w;
    }
    return total;
  };
  f32x4 y = sum(tile);
  if (up_tiles > 0) {
    const f32x4 o = sum(tile + up_tiles);
    const float g[4] = {round_to_elem(y.x), round_to_elem(y.y), round_to_elem(y.z), round_to_elem(y.w)};
    const float u[4] = {round_to_elem(o.x), round_to_elem(o.y), round_to_elem(o.z), round_to_elem(o.w)};
    y.x = (g[0] * (1.0f / (1.0f + expf(-g[0])))) * u[0];
    y.y = (g[1] * (1.0f / (1.0f + expf(-g[1])))) * u[1];
    y.z = (g[2] * (1.0f / (1.0f + expf(-g[2])))) * u[2];
    y.w = (g[3] * (1.0f / (1.0f + expf(-g[3])))) * u[3];
  }
  store_out4(out, ldo, mt * 16 + r16, tile * 16 + 4 * kg, M, N, y, out_vec_ok);
}

template <int MT>
static int launch_split(elem_t* out, const elem_t* act, const elem_t* w, int M, int rows, int K, int64_t lda, int64_t ldo,
                        int swiglu, float* workspace, int vec_ok, hipStream_t st) {
  const int ntiles16 = (rows + 15) / 16, nchunks = K / KC;
  f32x4* partial = reinterpret_cast<f32x4*>(workspace);
  // Eight waves a workgroup where that still leaves two workgroups or more per compute unit, else four
  // (64 rows, 4096 x 12288: 37.3 against 35.7 us; 6144 x 4096: 19.1 against 19.9 us; sixteen waves were slower).
  if ((int64_t)((ntiles16 + 7) / 8) * nchunks >= 2 * device_cus())
    gemm_split_kernel<MT, 8><<<dim3((ntiles16 + 7) / 8, nchunks), 512, 0, st>>>(partial, act, w, M, rows, K, lda, ntiles16);
  else
    gemm_split_kernel<MT, 4><<<dim3((ntiles16 + 3) / 4, nchunks), 256, 0, st>>>(partial, act, w, M, rows, K, lda, ntiles16);
  const int up_tiles = swiglu ? ntiles16 / 2 : 0;
  const int out_tiles = swiglu ? up_tiles : ntiles16;
  const int64_t threads = (int64_t)out_tiles * MT * 64;
  gemm_split_reduce_kernel<MT><<<(unsigned)((threads + 255) / 256), 256, 0, st>>>(out, partial, M, swiglu ? rows / 2 : rows, ldo,
                                                                                  nchunks, ntiles16, up_tiles, vec_ok);
  return vk_check_launch("gemm_split");
}
#endif

// ==================================================================== host
static int device_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (cus <= 0) cus = 256;
  }
  return cus;
}

// Waves a workgroup of the streaming kernels at up to 16 rows, for K of nchunks chunks.  Wave w takes the chunks
// w, w + waves, ...: with eight waves and ten chunks two waves have a second chunk and six wait for them at every
// tile's barrier, and with two chunks six of eight waves only take up room.  One chunk a wave where a workgroup
// can be that size (16-bit elements: up to 12 waves; the registers of 32-bit activations allow 8), measured on an
// MI355X at 8 rows: 34816 gate rows x 5120: 88.6 -> 80.0 us, 7168 x 5120: 23.8 -> 20.4, 2048 x 6144: 12.5 -> 11.2,
// 151936 x 1024: 103 -> 59, 151936 x 2048: 142 -> 116, 4096 x 1024: 5.5 -> 4.2.  More chunks than that: eight waves
// (ten or twelve without resident activations: 5120 x 17408 56.8 -> 66 us).
static int stream_waves(int nchunks) {
  if (nchunks <= 2) return 2;
  if (nchunks <= 4) return 4;
  if (nchunks <= 6) return nchunks;
  if (nchunks <= 8) return 8;
#ifdef VK_BF16
  if (nchunks <= 10) return 10;
  if (nchunks <= 12) return 12;
#endif
  return 8;
}

// Which kernel computes a product (speed only: all give the same bits).  Every threshold is a count of
// workgroups against the device's compute units (cus), or a count of 16-row activation tiles, or whether a
// wave's share of K fits its registers; none is a model's size.  With the workgroups a kernel would start:
//   wg16  = ceil(N / 16)   the streaming kernels (one 16-row weight tile a workgroup; two with kernel 7)
//   wg32, wg64, wg128      the kernel that shares activations through LDS (32, 64 or 128 weight rows a workgroup)
//   k_resident             K <= 8 chunks: each of a workgroup's 8 waves has one chunk, whose activations stay in registers
//
//   rows     condition                                         kernel
//   1..16                                                      1   streaming
//   17..32   16-bit, K whole chunks, k_resident,               11  streaming, both activation tiles of a wave's chunk in
//            wg16 >= 1.5 cus                                       registers (32 rows, 24576 x 4096: 53 -> 44 us)
//   17..64   K whole chunks:
//              wg128 >= 0.75 cus                               10  128 weight rows a workgroup: the activations that every
//                                                                  workgroup reads are half the weight bytes (64 rows, 51200 x
//                                                                  5120: 158 -> 127 us)
//              wg64 >= 0.5 cus                                 8   64 weight rows a workgroup
//              rows > 32, wg32 <= 0.5 cus, and rows > 40 or    12  so few weight rows that workgroups of 32 leave half the units
//                not k_resident                                    idle: two blocks of 32 rows side by side (64 rows, 4096 x
//                                                                  12288: 55 -> 45 us)
//              rows > 40                                       9   32 weight rows a workgroup
//              k_resident or wg16 <= cus                       7 / 1  streaming, two weight tiles a workgroup from wg16 >= 1.5 cus
//              else                                            9   the streaming kernel would need a second pass for a few tiles
//                                                                  (32 rows, 5120 x 17408: 111 -> 65 us)
//   17..64   K not in whole chunks                             2 (rows > 32 and wg128 >= 0.5 cus), else 7 / 1 as above
//   65..256  K whole chunks, wg128 < 0.5 cus:                      the tile kernel would have a workgroup or less per unit, each
//                                                                  walking all of K alone (4096 x 12288: 170 us at any of these
//                                                                  rows); the LDS-sharing kernel in blocks of 64 rows fills the
//                                                                  chip (100 rows: 51 us, 200 rows: 82 us)
//              wg64 >= 0.5 cus                                 8 up to three blocks, else 2
//              two blocks                                      9 (wg32 <= 0.5 cus) or 8
//              else                                            2 (k_resident and wg16 >= 1.5 cus) or 8
//   more                                                       2   the pipelined tile kernel
// With a workspace the products of up to 64 rows that vk_gemm_split_preferred names go through chunk sums
// instead (the caller's choice: vk_gemm_split).
static int choose_gemm_kernel(int M, int N, int K) {
  const int cus = device_cus();
  const int wg16 = (N + 15) / 16, wg32 = (N + 31) / 32, wg64 = (N + 63) / 64, wg128 = (N + 127) / 128;
  const bool whole = K % KC == 0, k_resident = K <= SK_WAVES * KC;
  const bool many16 = 2 * wg16 >= 3 * cus;
  if (M <= 16) return 1;
  if (M <= 32 && whole && k_resident && many16 && sizeof(elem_t) == 2) return 11;
  if (M <= 64 && whole) {
    if (4 * wg128 >= 3 * cus) return 10;
    if (2 * wg64 >= cus) return 8;
    if (M > 32 && 2 * wg32 <= cus && (M > 40 || !k_resident)) return 12;
    if (M > 40) return 9;
    if (k_resident || wg16 <= cus) return many16 ? 7 : 1;
    return 9;
  }
  if (M <= 64) return (2 * wg128 >= cus && M > 32) ? 2 : (many16 ? 7 : 1);
  if (M <= 256 && whole && 2 * wg128 < cus) {
    const int blocks = (M + 63) / 64;
    if (2 * wg64 >= cus) return blocks <= 3 ? 8 : 2;
    if (blocks == 2) return 2 * wg32 <= cus ? 9 : 8;
    return (k_resident && many16) ? 2 : 8;
  }
  return 2;
}

// How many 16-row weight fragments a wave of the tile kernel takes (a workgroup: 32 of them in weight rows).  The
// kernel's time goes in rounds of the workgroups that the device holds at once, two per compute unit: a last round
// that is nearly empty costs almost a whole one (0.72 of one up to half full, where every workgroup has its unit
// to itself).  A round costs 0.9, 1 and 1.25 times the square tile's with 96, 128 and 160 weight rows (measured at
// 1,024 to 8,192 rows on 4,096 to 10,240 weight rows); another width is taken when that makes the sum 3 % smaller:
// 5,120 weight rows at 2,048 rows are 1.25 rounds of 128 or one of 160 (5,120 x 5,120: 121 -> 93 us, 5,120 x
// 17,408: 452 -> 337, 5,120 x 25,600: 705 -> 481), 6,144 weight rows at 1,024 rows 0.75 rounds of 128 or one of 96
// (62 -> 53 us).
static int pipe_fragments_by_rounds(int M, int N) {
  static const double round_cost[6] = {0, 0, 0, 0.9, 1.0, 1.25};
  const double slots = 2.0 * device_cus();
  const int mb = (M + 127) / 128;
  auto estimate = [&](int f) {
    const double rounds = (double)((N + 32 * f - 1) / (32 * f)) * mb / slots;
    const double whole = std::floor(rounds), part = rounds - whole;
    return round_cost[f] * (whole + (part == 0 ? 0.0 : (part <= 0.5 ? 0.72 : 1.0)));
  };
  int best = 4;
  double least = 0.97 * estimate(4);
  for (int f : {3, 5}) {
    const double e = estimate(f);
    if (e < least) {
      least = e;
      best = f;
    }
  }
  return best;
}

extern "C" {

// kernel: 0 = choose by size, 1 = skinny (M <= 64), 2 = tiled (pipelined if K allows), 3 = tiled through
// registers, 4..6 = pipelined with 2..4 stages, 7 = skinny with two weight tiles per workgroup where it has
// such a variant, 8, 9 and 10 = activations shared through LDS with 64, 32 and 128 weight rows per workgroup
// (17 to 512 rows, in blocks of 64 rows), 11 = skinny with two activation tiles resident in registers (17 to
// 32 rows of 16-bit elements, K <= 4096), 12 = as 9 in blocks of 32 rows, 13, 15 and 16 = pipelined with 64, 96
// and 160 weight rows per workgroup (14 is the callers' name for the route through chunk sums); for measurements and tests.  The result does not depend on the choice.
int vk_gemm(elem_t* out, const elem_t* act, const elem_t* w, int M, int N, int K, int64_t lda, int64_t ldo,
            int kernel, hipStream_t st) {
  VK_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  VK_REQUIRE(K % VK_VEC == 0, "gemm: K=%d must be a multiple of %d for this element type", K, VK_VEC);
  VK_REQUIRE(lda >= K && lda % VK_VEC == 0, "gemm: activation row stride %lld must be >= K and a multiple of %d",
             (long long)lda, VK_VEC);
  VK_REQUIRE(ldo >= N, "gemm: output row stride %lld is smaller than N=%d", (long long)ldo, N);
  VK_REQUIRE(((uintptr_t)act % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm: operands must be 16-byte aligned");
  VK_REQUIRE(kernel >= 0 && kernel <= 16 && kernel != 14, "gemm: unknown kernel %d", kernel);
  if (M == 0) return 0;
  const int vec_ok = (ldo % 4 == 0) && ((uintptr_t)out % 16 == 0);
  const bool by_size = kernel == 0;
  if (kernel == 0) kernel = choose_gemm_kernel(M, N, K);
  if (kernel == 12) {      // 32 weight rows per workgroup, four chunks in work, blocks of 32 rows
    VK_REQUIRE(M > 16 && M <= 512 && K % KC == 0, "gemm: the mid kernel takes 17 to 512 rows and K a multiple of %d", KC);
    return launch_mid<2, 4>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
  }
  if (kernel >= 8 && kernel <= 10) {
    VK_REQUIRE(M > 16 && M <= 512 && K % KC == 0, "gemm: the mid kernel takes 17 to 512 rows and K a multiple of %d", KC);
    const int mt = M > 64 ? 4 : (M + 15) / 16;       // more than 64 rows: blocks of 64
    if (kernel == 10) {     // 128 weight rows per workgroup, every wave all chunks of its tile
      if (mt == 2) return launch_mid<2, 1>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
      return launch_mid<4, 1>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
    }
    if (kernel == 8) {      // 64 weight rows per workgroup, two chunks in work
      if (mt == 2) return launch_mid<2, 2>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
      if (mt == 3) return launch_mid<3, 2>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
      return launch_mid<4, 2>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
    }
    // 32 weight rows per workgroup, four chunks in work
    if (mt == 2) return launch_mid<2, 4>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
    if (mt == 3) return launch_mid<3, 4>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
    return launch_mid<4, 4>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
  }
  if (kernel == 11)
    VK_REQUIRE(M > 16 && M <= 32 && K % KC == 0 && K <= SK_WAVES * KC && sizeof(elem_t) == 2,
               "gemm: resident activations of two tiles need 17 to 32 rows of 16-bit elements and K a multiple of %d up to %d", KC, SK_WAVES * KC);
  if (kernel == 1 || kernel == 7 || kernel == 11) {
    VK_REQUIRE(M <= 64, "gemm: the skinny kernel takes at most 64 rows, got %d", M);
    const int mt = (M + 15) / 16;
    const unsigned grid = (unsigned)((N + 15) / 16);
    if (K % KC == 0) {
#define STW(MT, W, RC, NT, NW)                                                                            \
  do {                                                                                                    \
    static int resident = 0; /* workgroups of this kernel that the device holds at once */               \
    if (resident == 0) {                                                                                  \
      int dev = 0, cus = 0, per_cu = 0;                                                                   \
      (void)hipGetDevice(&dev);                                                                           \
      (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);                      \
      (void)hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gemm_stream_kernel<MT, W, RC, NT, NW>,  \
                                                         64 * NW, 0);                                     \
      resident = (cus > 0 ? cus : 256) * (per_cu > 0 ? per_cu : 1);                                       \
    }                                                                                                     \
    const unsigned groups = (unsigned)((N + 16 * NT - 1) / (16 * NT));                                    \
    gemm_stream_kernel<MT, W, RC, NT, NW><<<groups < (unsigned)resident ? groups : (unsigned)resident,    \
                                             64 * NW, 0, st>>>(out, act, w, M, N, K, lda, ldo, vec_ok);   \
  } while (0)
#define ST(MT, W, RC, NT) STW(MT, W, RC, NT, SK_WAVES)
      if (mt == 1) {
        // A few weight tiles more than workgroups in flight (one per compute unit) would mean a second
        // pass of a few: two tiles a workgroup then finish sooner (16 rows, 5120 x 25600: 111 -> 86 us),
        // unless one chunk a wave keeps the activations in registers (6144 x 4096: 12.6 against 15.7 us).
        const int cus = device_cus();
        const int tiles16 = (N + 15) / 16;
        // One chunk a wave, its activations in registers, wherever a workgroup can have as many waves as K has
        // chunks (stream_waves): no wave then waits at the round's barrier for one that has a second chunk.
        const int nw = kernel == 7 ? SK_WAVES : stream_waves(K / KC);
        if (nw == 2) STW(1, 8, 1, 1, 2);
        else if (nw == 4) STW(1, 8, 1, 1, 4);
        else if (nw == 5) STW(1, 8, 1, 1, 5);
        else if (nw == 6) STW(1, 8, 1, 1, 6);
#ifdef VK_BF16
        else if (nw == 10) STW(1, 8, 1, 1, 10);
        else if (nw == 12) STW(1, 8, 1, 1, 12);
#endif
        else
        if (kernel == 7 || (by_size && K > SK_WAVES * KC && tiles16 > cus && 2 * tiles16 <= 3 * cus)) ST(1, 8, 0, 2);
        else if (K <= SK_WAVES * KC) ST(1, 8, 1, 1);
#ifdef VK_BF16
        // Two chunks a wave are 128 registers of activations (16 rows, 34816 x 5120: 118 -> 87 us);
        // three did not fit beside the rest and were slower than none (4096 x 12288: 29 -> 36 us).
        else if (K <= 2 * SK_WAVES * KC) ST(1, 8, 2, 1);
#endif
        else ST(1, 8, 0, 1);
      }
      else if (mt == 2) {
#ifdef VK_BF16
        if (kernel == 11) ST(2, 8, 1, 1);
        else
#endif
        if (kernel == 7) ST(2, 4, 0, 2);
        else ST(2, 8, 0, 1);
      }
      else if (mt == 3) { if (kernel == 7) ST(3, 4, 0, 2); else ST(3, 4, 0, 1); }
      else { if (kernel == 7) ST(4, 4, 0, 2); else ST(4, 4, 0, 1); }
#undef ST
#undef STW
      return vk_check_launch("gemm_stream");
    }
#define SK(MT, W) gemm_skinny_kernel<MT, W><<<grid, 64 * SK_WAVES, 0, st>>>(out, act, w, M, N, K, lda, ldo, vec_ok)
    // Few weight rows leave one workgroup per compute unit: a deeper window keeps its memory pipe full.
    if (mt == 1) { if (N <= 8192) SK(1, 16); else SK(1, 8); }
    else if (mt == 2) SK(2, 8);
    else if (mt == 3) SK(3, 4);
    else SK(4, 4);
#undef SK
    return vk_check_launch("gemm_skinny");
  }
  const bool k_whole = K % (2 * VK_SLAB) == 0;
  if (kernel == 3) return launch_tiled<4, 4>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
  if (kernel == 4 && k_whole) return launch_pipe<2>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
  if (kernel == 5 && k_whole) return launch_pipe<3>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
  if (kernel == 6 && k_whole) return launch_pipe<4>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
  // Two stages of 32 KB leave room for two workgroups per compute unit, which hides more latency than a third stage.
  if (k_whole) {
    // No more 128 x 128 tiles than compute units: 64 weight rows a workgroup, twice as many of them
    // (512 rows, 4096 x 12288: 163 -> 145 us; a workgroup alone on its compute unit is bound by what one
    // compute unit can read, whatever the number of stages).
    const int64_t tiles = (int64_t)((N + 127) / 128) * ((M + 127) / 128);
    if (kernel == 13 || (by_size && tiles <= device_cus())) return launch_pipe<2, false, 2>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
    const int fragments = kernel == 15 ? 3 : (kernel == 16 ? 5 : (by_size ? pipe_fragments_by_rounds(M, N) : 4));
    if (fragments == 3) return launch_pipe<2, false, 3>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
    if (fragments == 5) return launch_pipe<2, false, 5>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
    return launch_pipe<2>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
  }
  return launch_tiled<4, 4>(out, act, w, M, N, K, lda, ldo, vec_ok, st);
}

// 1 if vk_gemm_swiglu takes these sizes (the caller otherwise runs vk_gemm and vk_swiglu, with the same result).
// 1: the streaming kernel (few rows), 2: the pipelined tile kernel (many rows), 3: the kernel for 17 to 64
// rows that shares activations through LDS, 0: none.
int vk_gemm_swiglu_supported(int M, int I, int K) {
  if (M >= 1 && M <= 16 && I > 0 && K % KC == 0 && K <= SK_WAVES * KC) return 1;
#ifdef VK_BF16
  if (M > 16 && M <= 32 && I > 0 && K % KC == 0 && K <= SK_WAVES * KC) return 1;    // two activation tiles in registers
  if (M >= 1 && M <= 16 && I > 0 && K % KC == 0 && K <= 2 * SK_WAVES * KC) return 1;   // two chunks a wave
#endif
  if (M > 64 && I > 0 && K % (2 * VK_SLAB) == 0) return 2;
  if (M > 16 && M <= 64 && I > 0 && K % KC == 0) return 3;      // activations shared through LDS
  return 0;
}

// out[M, I] = silu(act w_gate^T) * (act w_up^T), w = [gate rows; up rows] of shape [2I, K].
int vk_gemm_swiglu(elem_t* out, const elem_t* act, const elem_t* w, int M, int I, int K, int64_t lda, int64_t ldo,
                   hipStream_t st) {
  const int how = vk_gemm_swiglu_supported(M, I, K);
  VK_REQUIRE(how != 0, "gemm_swiglu: sizes M=%d I=%d K=%d are not supported", M, I, K);
  VK_REQUIRE(lda >= K && lda % VK_VEC == 0 && ldo >= I, "gemm_swiglu: bad row strides");
  VK_REQUIRE(((uintptr_t)act % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_swiglu: operands must be 16-byte aligned");
  if (how == 2)
    return launch_pipe<2, true>(out, act, w, M, I, K, lda, ldo, (ldo % 4 == 0) && ((uintptr_t)out % 16 == 0), st);
  if (how == 3) {
    const int ok4 = (ldo % 4 == 0) && ((uintptr_t)out % 16 == 0);
    // Gate tiles per workgroup: of four, three and two, the number whose workgroups fill the compute units
    // best, a workgroup per unit at a time; the larger one where two fill them alike.  64 rows, K = 4096:
    // 12288 gate rows (192, 256, 384 workgroups) 55.4, 49.7, 58.5 us; 8192 gate rows (128, 171, 256) 52.8, 47.0,
    // 41.6 us; 17408 gate rows at K = 5120 (272, 363, 544) 127.5, 108.4, 123.2 us.
    const int tiles = (I + 15) / 16, cus = device_cus();
    int gt = 4;
    double best = 0.0;
    for (int g = 4; g >= 2; --g) {
      const int wgs = (tiles + g - 1) / g;
      const double filled = (double)wgs / ((double)((wgs + cus - 1) / cus) * cus);
      if (filled > best + 1e-9) { best = filled; gt = g; }
    }
    if (M <= 32) {
      if (gt == 3) return launch_mid<2, 1, true, 3>(out, act, w, M, I, K, lda, ldo, ok4, st);
      if (gt == 2) return launch_mid<2, 1, true, 2>(out, act, w, M, I, K, lda, ldo, ok4, st);
      return launch_mid<2, 1, true>(out, act, w, M, I, K, lda, ldo, ok4, st);
    }
    if (gt == 3) return launch_mid<4, 1, true, 3>(out, act, w, M, I, K, lda, ldo, ok4, st);
    if (gt == 2) return launch_mid<4, 1, true, 2>(out, act, w, M, I, K, lda, ldo, ok4, st);
    return launch_mid<4, 1, true>(out, act, w, M, I, K, lda, ldo, ok4, st);
  }
  const int ntiles = (I + 15) / 16;
  const int vec_ok = (ldo % 4 == 0) && ((uintptr_t)out % 16 == 0);
#define SWIGLU_STREAMW(W, MT, RC, NW)                                                                       \
  do {                                                                                                     \
    static int resident = 0;                                                                               \
    if (resident == 0) {                                                                                   \
      int dev = 0, cus = 0, per_cu = 0;                                                                    \
      (void)hipGetDevice(&dev);                                                                            \
      (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);                       \
      (void)hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gemm_stream_swiglu_kernel<W, MT, RC, NW>, \
                                                         64 * NW, 0);                                      \
      resident = (cus > 0 ? cus : 256) * (per_cu > 0 ? per_cu : 1);                                        \
    }                                                                                                      \
    gemm_stream_swiglu_kernel<W, MT, RC, NW><<<ntiles < resident ? ntiles : resident, 64 * NW, 0, st>>>(   \
        out, act, w, M, I, K, lda, ldo, vec_ok);                                                           \
  } while (0)
#define SWIGLU_STREAM(W, MT, RC) SWIGLU_STREAMW(W, MT, RC, SK_WAVES)
  const int nw = M <= 16 ? stream_waves(K / KC) : SK_WAVES;       // as in vk_gemm
  if (nw == 2) SWIGLU_STREAMW(8, 1, 1, 2);
  else if (nw == 4) SWIGLU_STREAMW(8, 1, 1, 4);
  else if (nw == 5) SWIGLU_STREAMW(8, 1, 1, 5);
  else if (nw == 6) SWIGLU_STREAMW(8, 1, 1, 6);
#ifdef VK_BF16
  else if (nw == 10) SWIGLU_STREAMW(8, 1, 1, 10);
  else if (nw == 12) SWIGLU_STREAMW(8, 1, 1, 12);
#endif
  else
#ifdef VK_BF16
  if (M > 16) SWIGLU_STREAM(4, 2, 1);
  else if (K > SK_WAVES * KC) SWIGLU_STREAM(4, 1, 2);
  else
#endif
    SWIGLU_STREAM(8, 1, 1);
#undef SWIGLU_STREAM
#undef SWIGLU_STREAMW
  return vk_check_launch("gemm_swiglu");
}


// float32 elements of workspace that vk_gemm_split needs for these sizes, or 0 if it does not take them:
// up to 64 rows of 16-bit elements, K in whole chunks; rows: weight rows (with swiglu: gate and up rows
// together, an even number of 16-row tiles).
int64_t vk_gemm_split_floats(int M, int rows, int K, int swiglu) {
#ifdef VK_BF16
  if (M <= 0 || M > 64 || rows <= 0 || K <= 0 || K % KC != 0) return 0;
  if (swiglu && rows % 32 != 0) return 0;
  const int mt = (M + 15) / 16;
  return (int64_t)(K / KC) * ((rows + 15) / 16) * mt * 256;
#else
  (void)M; (void)rows; (void)K; (void)swiglu;
  return 0;
#endif
}

// 1 if the route through chunk sums is the faster one for these sizes (measured on an MI355X).  Not with the
// activation folded in (24576 x 4096 at 64 rows: 60 -> 62 us), not for matrices of less than 64 KB per compute
// unit (1000 x 1024 at 32 rows: 4.8 -> 6.5 us), and not where workgroups of 128 weight rows are a quarter of the
// compute units or more: the other kernels then have workgroups enough, and the chunk sums would be a large
// share of the traffic.
//   17 to 64 rows: always then (64 rows: 4096 x 12288 45 -> 32 us, 6144 x 4096 20.6 -> 18.2, 4096 x 4096 16.0 -> 13.8;
//     32 rows: 41 -> 27, 17.8 -> 14.7, 13.4 -> 11.7 us).
//   Up to 16 rows the streaming kernel is the other choice.  With `fill` the share of the compute units that
//   its last round of one workgroup per 16 weight rows keeps busy:
//     K of more than 16 chunks (its waves read their activations again for every chunk): when fill < 0.9
//       (8 rows: 5120 x 17408 56.8 -> 41.7 us, 5120 x 25600 80.8 -> 57.8, 2560 x 9728 19.7 -> 15.3) or from 8 rows on
//       (4096 x 12288, fill 1: 1 row 23.0 -> 24.5 us, 4 rows 24.7 -> 24.5, 8 rows 27.2 -> 23.9, 16 rows 29.3 -> 24.0);
//     K of 9 to 16 chunks: when fill < 0.7 (8 rows: 5120 x 5120 18.5 -> 16.6 us, 5120 x 8192 25.9 -> 24.0, 2048 x
//       6144 11.2 -> 9.6; but 7168 x 5120, fill 0.88, 19.1 -> 21.2);
//     K of up to 8 chunks: never (4096 x 4096 9.1 -> 10.3 us, 2560 x 4096, fill 0.63, 8.3 -> 9.2).
int vk_gemm_split_preferred(int M, int rows, int K, int swiglu) {
  if (swiglu || vk_gemm_split_floats(M, rows, K, swiglu) == 0) return 0;
  const int cus = device_cus();
  const int64_t bytes = (int64_t)rows * K * (int64_t)sizeof(elem_t);
  if (bytes < (int64_t)cus * 65536 || 4 * ((rows + 127) / 128) > cus) return 0;
  if (M > 16) return 1;
  const int nchunks = K / KC, tiles16 = (rows + 15) / 16;
  const int rounds = (tiles16 + cus - 1) / cus;
  const bool fill_below_09 = 10 * tiles16 < 9 * rounds * cus, fill_below_07 = 10 * tiles16 < 7 * rounds * cus;
  if (nchunks > 2 * SK_WAVES) return fill_below_09 || M >= 8;
  return nchunks > SK_WAVES && fill_below_07;
}

// out = act w^T (swiglu 0: w [rows, K], out [M, rows]) or silu(act w_gate^T) * (act w_up^T) (swiglu 1:
// w = [gate rows; up rows], out [M, rows / 2]), through chunk sums in a workspace: the bits of vk_gemm and
// vk_gemm_swiglu.  Calls that overlap in time need workspaces of their own.
int vk_gemm_split(elem_t* out, const elem_t* act, const elem_t* w, int M, int rows, int K, int64_t lda, int64_t ldo,
                  int swiglu, float* workspace, int64_t workspace_floats, hipStream_t st) {
  const int64_t need = vk_gemm_split_floats(M, rows, K, swiglu);
  VK_REQUIRE(need > 0, "gemm_split: sizes M=%d rows=%d K=%d are not supported", M, rows, K);
  VK_REQUIRE(workspace != nullptr && workspace_floats >= need && ((uintptr_t)workspace % 16) == 0,
             "gemm_split: a 16-byte aligned workspace of %lld floats is needed", (long long)need);
  const int out_cols = swiglu ? rows / 2 : rows;
  VK_REQUIRE(lda >= K && lda % VK_VEC == 0 && ldo >= out_cols, "gemm_split: bad row strides");
  VK_REQUIRE(((uintptr_t)act % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_split: operands must be 16-byte aligned");
#ifdef VK_BF16
  const int vec_ok = (ldo % 4 == 0) && ((uintptr_t)out % 16 == 0);
  const int mt = (M + 15) / 16;
  if (mt == 1) return launch_split<1>(out, act, w, M, rows, K, lda, ldo, swiglu, workspace, vec_ok, st);
  if (mt == 2) return launch_split<2>(out, act, w, M, rows, K, lda, ldo, swiglu, workspace, vec_ok, st);
  if (mt == 3) return launch_split<3>(out, act, w, M, rows, K, lda, ldo, swiglu, workspace, vec_ok, st);
  return launch_split<4>(out, act, w, M, rows, K, lda, ldo, swiglu, workspace, vec_ok, st);
#else
  (void)out; (void)st;
  return vk_fail("gemm_split: built for 16-bit elements only");
#endif
}

}  // extern "C"
