// A routed feed-forward: a float32 router with softmax scores and a choice of the `top` best
// experts per token, the (token, choice) pairs put in the order of their experts, the experts'
// products over those runs of rows, and the weighted sum per token.
#include "common.h"
#include "gemm_tiles.h"

#include <math.h>

__device__ inline float moe_gelu(float z, int kind) {
  if (kind == 0) return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
  return 0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
}

// What the products' epilogues do with their sums (`act`): -1 nothing; 0, 1 the exact gelu and its tanh
// form on every sum; from 2 on a gated unit over neighbouring columns, out[j] = g(sum[2j]) * sum[2j + 1]
// with g silu (2), the tanh form of gelu (3) or the exact gelu (4): the weight's rows interleave gate
// and up, the result has half the columns, and both sums enter unrounded.
#define MOE_ACT_GATED 2
#define MOE_ACT_MOST 4
__device__ inline float moe_gated(float g, float u, int act) {
  if (act == MOE_ACT_GATED) return g / (1.f + expf(-g)) * u;
  return moe_gelu(g, act == 3 ? 1 : 0) * u;
}

// ---------------------------------------------------------------------------
// The router's choice. One wavefront per token, from its float32 logits z (E numbers, a token's
// `row_stride` apart). `mode` 0: s = softmax(z) over all E experts, then `top` times the largest
// remaining score (the lowest index among equals); weight_k = s_k / (sum of the chosen s + 1e-20).
// `mode` 1: s = sigmoid(z), each expert for itself; the `top` largest are those with the largest z
// (chosen by z, which still tells experts apart where the sigmoid has run into 1); weight_k = s_k as it
// is. `mode` 2: s = sigmoid(z); the choice goes by c = s + correction[e] and only among the experts of
// `keep` of the `groups` equal groups of neighbours, those whose two largest c sum highest (the lowest
// group among equals; the others' c count as minus infinity); weight_k = s_k as it is, without the
// correction. Every lane holds every reduced number; what one lane writes to shared memory and
// another reads is separated by the wavefront's barrier.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_pick_kernel(const float* __restrict__ logits, long row_stride, int n_tokens,
                                                       int E, int top, int mode, const float* __restrict__ correction,
                                                       int groups, int keep, int* __restrict__ chosen,
                                                       float* __restrict__ weights) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x / Q3_WAVE, lane = threadIdx.x % Q3_WAVE;
  const int t = blockIdx.x * (blockDim.x / Q3_WAVE) + wave;
  if (t >= n_tokens) return;
  float* z = smem + (size_t)wave * (E + top + groups);     // the wavefront's scores, then the chosen ones, then the groups'
  float* picked = z + E;
  float* group_score = picked + top;
  const float* src = logits + (size_t)t * row_stride;
  float total = 1.f;
  if (mode == 0) {
    float biggest = -INFINITY;
    for (int e = lane; e < E; e += Q3_WAVE) biggest = fmaxf(biggest, src[e]);
    biggest = wave_max(biggest);
    total = 0.f;
    for (int e = lane; e < E; e += Q3_WAVE) {
      const float p = expf(src[e] - biggest);
      z[e] = p;
      total += p;
    }
    total = wave_sum(total);
  } else if (mode == 1) {
    for (int e = lane; e < E; e += Q3_WAVE) z[e] = src[e];
  } else {
    for (int e = lane; e < E; e += Q3_WAVE) z[e] = 1.f / (1.f + expf(-src[e])) + correction[e];
  }
  __builtin_amdgcn_wave_barrier();
  if (mode == 2 && keep < groups) {
    const int size = E / groups;
    for (int g = lane; g < groups; g += Q3_WAVE) {          // a group a lane: the sum of its two largest
      float first = -INFINITY, second = -INFINITY;
      for (int i = 0; i < size; ++i) {
        const float c = z[g * size + i];
        if (c > first) {
          second = first;
          first = c;
        } else if (c > second) {
          second = c;
        }
      }
      group_score[g] = size > 1 ? first + second : first;
    }
    __builtin_amdgcn_wave_barrier();
    // an expert stays if fewer than `keep` groups stand before its own (a higher score, or an equal one
    // and a lower number): every lane ranks its expert's group against all of them, no round of maxima
    for (int e = lane; e < E; e += Q3_WAVE) {
      const int g = e / size;
      const float own = group_score[g];
      int before = 0;
      for (int j = 0; j < groups; ++j) {
        const float other = group_score[j];
        before += (other > own || (other == own && j < g)) ? 1 : 0;
      }
      if (before >= keep) z[e] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
  const float nothing = mode == 0 ? -1.f : -INFINITY;     // below every score that can still be chosen
  float picked_sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = nothing;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += Q3_WAVE) {
      const float p = z[e];
      if (p > best) {
        best = p;
        at = e;
      }
    }
#pragma unroll
    for (int off = Q3_WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, Q3_WAVE);
      const int oa = __shfl_xor(at, off, Q3_WAVE);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (at >= E) at = 0;          // logits that are no numbers: stay inside the operands
    const float score = mode == 0 ? best / total : 1.f / (1.f + expf(-(mode == 1 ? best : src[at])));
    picked_sum += score;
    __builtin_amdgcn_wave_barrier();
    picked[k] = score;
    z[at] = mode == 0 ? -2.f : -INFINITY;               // taken
    if (lane == 0) chosen[(size_t)t * top + k] = at;
    __builtin_amdgcn_wave_barrier();
  }
  const float inv = mode == 0 ? 1.f / (picked_sum + 1e-20f) : 1.f;
  for (int k = lane; k < top; k += Q3_WAVE) weights[(size_t)t * top + k] = picked[k] * inv;
}

// ---------------------------------------------------------------------------
// Pairs in the order of their experts. One block. `chosen` (P) names each pair's expert.
//   offsets[e] .. offsets[e+1]: the slots of expert e;  pair_of_slot[slot] = pair;
//   slot_of_pair[pair] = slot;  tiles of `tile_rows` slots that never cross an expert's end:
//   tile_expert[i], tile_first[i] (first slot), n_tiles[0].
// Which slot of its expert's run a pair gets depends on the order in which threads arrive; a
// row's result does not depend on its slot.
// ---------------------------------------------------------------------------
__global__ void moe_align_kernel(const int* __restrict__ chosen, int P, int E, int tile_rows,
                                 int* __restrict__ offsets, int* __restrict__ pair_of_slot,
                                 int* __restrict__ slot_of_pair, int* __restrict__ tile_expert,
                                 int* __restrict__ tile_first, int* __restrict__ n_tiles) {
  extern __shared__ int counts[];   // [E] counts, then [E] cursors
  int* cursor = counts + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = chosen[p];
    if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = at;
      cursor[e] = at;
      for (int r = 0; r < counts[e]; r += tile_rows) {
        tile_expert[tiles] = e;
        tile_first[tiles] = at + r;
        ++tiles;
      }
      at += counts[e];
    }
    offsets[E] = at;
    n_tiles[0] = tiles;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = chosen[p];
    if (e >= 0 && e < E) {
      const int slot = atomicAdd(&cursor[e], 1);
      pair_of_slot[slot] = p;
      slot_of_pair[p] = slot;
    }
  }
}

// ---------------------------------------------------------------------------
// The experts' products over the sorted slots, float32 multiply-adds, any sizes:
//   out[slot, n] = act(sum_k x[src(slot), k] * w[e, n, k]),  e the expert of the slot's tile,
//   src(slot) = pair_of_slot[slot] / pairs_per_row if `gather` else slot.
// A block: one tile of 16 slots, 64 output columns; x and w pass shared memory in slices of 32 k.
// ---------------------------------------------------------------------------
#define MOE_BM 16
#define MOE_BN 64
#define MOE_BK 32

template <typename T>
__global__ __launch_bounds__(256) void moe_linear_kernel(const T* __restrict__ x, const int* __restrict__ pair_of_slot,
                                                         int gather, int pairs_per_row, const T* __restrict__ w,
                                                         T* __restrict__ out, const int* __restrict__ tile_expert,
                                                         const int* __restrict__ tile_first,
                                                         const int* __restrict__ offsets,
                                                         const int* __restrict__ n_tiles, int N, int K, int act) {
  __shared__ float xs[MOE_BM][MOE_BK + 1];
  __shared__ float ws[MOE_BN][MOE_BK + 1];
  __shared__ int src_row[MOE_BM];
  const int tile = blockIdx.x;
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile];
  const int first = tile_first[tile];
  const int rows = min(MOE_BM, offsets[e + 1] - first);
  const int n0 = blockIdx.y * MOE_BN;
  const int t = threadIdx.x;
  if (t < MOE_BM) src_row[t] = t < rows ? (gather ? pair_of_slot[first + t] / pairs_per_row : first + t) : -1;
  __syncthreads();
  const int r = t >> 4, c = t & 15;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const T* we = w + (size_t)e * N * K;
  for (int k0 = 0; k0 < K; k0 += MOE_BK) {
    for (int idx = t; idx < MOE_BM * MOE_BK; idx += 256) {
      const int m = idx / MOE_BK, kk = idx - m * MOE_BK;
      const int s = src_row[m];
      xs[m][kk] = (s >= 0 && k0 + kk < K) ? to_float(x[(size_t)s * K + k0 + kk]) : 0.f;
    }
    for (int idx = t; idx < MOE_BN * MOE_BK; idx += 256) {
      const int n = idx / MOE_BK, kk = idx - n * MOE_BK;
      ws[n][kk] = (n0 + n < N && k0 + kk < K) ? to_float(we[(size_t)(n0 + n) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < MOE_BK; ++kk) {
      const float a = xs[r][kk];
      // a gated unit wants a thread's four columns side by side; every sum's order over k is the same either way
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] += a * ws[act >= MOE_ACT_GATED ? 4 * c + j : c + 16 * j][kk];
    }
    __syncthreads();
  }
  if (r >= rows) return;
  if (act >= MOE_ACT_GATED) {
#pragma unroll
    for (int j = 0; j < 4; j += 2) {
      const int n = n0 + 4 * c + j;
      if (n + 1 < N) out[(size_t)(first + r) * (N / 2) + n / 2] = from_float<T>(moe_gated(acc[j], acc[j + 1], act));
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + c + 16 * j;
    if (n < N) out[(size_t)(first + r) * N + n] = from_float<T>(act >= 0 ? moe_gelu(acc[j], act) : acc[j]);
  }
}

// ---------------------------------------------------------------------------
// The same products on the matrix cores (v_mfma_f32_16x16x32_bf16): bfloat16, K a multiple of 32.
// out^T (columns x slots) = W_e (columns x K) . x^T (K x slots): 16 weight rows are the first
// operand, 16 slots' rows of x the second, both straight from memory (a lane reads 16 bytes of
// one row per step of 32 k). A tile has up to 64 slots (four second operands, of which those
// beyond the tile's rows are skipped); a block's four wavefronts each own NS slabs of 16 output
// columns, so every x operand serves NS matrix instructions and every weight operand up to four.
// A lane ends up with four consecutive columns of one slot.
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float moe_f32x4_t;
union MoePack {
  uint4 u;
  moe_bf16x8_t v;
};
#define MMA_TM 64
#define MMA_MT 4

template <int NS>
__global__ __launch_bounds__(256) void moe_linear_mma_kernel(
    const bf16_t* __restrict__ x, const int* __restrict__ pair_of_slot, int gather, int pairs_per_row,
    const bf16_t* __restrict__ w, bf16_t* __restrict__ out, const int* __restrict__ tile_expert,
    const int* __restrict__ tile_first, const int* __restrict__ offsets, const int* __restrict__ n_tiles, int N, int K,
    int act) {
  const int tile = blockIdx.x;
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile];
  const int first = tile_first[tile];
  const int rows = min(MMA_TM, offsets[e + 1] - first);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const bf16_t* xr[MMA_MT];
#pragma unroll
  for (int mt = 0; mt < MMA_MT; ++mt) {
    const int m = 16 * mt + col;
    xr[mt] = nullptr;
    if (m < rows) {
      const int src = gather ? pair_of_slot[first + m] / pairs_per_row : first + m;
      xr[mt] = x + (size_t)src * K + 8 * grp;
    }
  }
  const int n_base = (blockIdx.y * 4 + wave) * (16 * NS);
  if (n_base >= N) return;
  const bf16_t* wr[NS];
#pragma unroll
  for (int ns = 0; ns < NS; ++ns) {
    const int n = n_base + 16 * ns + col;
    wr[ns] = n < N ? w + ((size_t)e * N + n) * K + 8 * grp : nullptr;
  }
  moe_f32x4_t acc[MMA_MT][NS];
#pragma unroll
  for (int mt = 0; mt < MMA_MT; ++mt)
#pragma unroll
    for (int ns = 0; ns < NS; ++ns) acc[mt][ns] = moe_f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int row_blocks = (rows + 15) >> 4;          // the same for every lane
  // U steps of 32 k are asked for together before their matrix instructions run. One slab a
  // wavefront is the case of few rows, where the weights stream from memory and what counts is
  // how many loads are on their way.
  constexpr int U = NS == 1 ? 4 : 2;
  for (int k0 = 0; k0 < K; k0 += 32 * U) {
    MoePack a[U][NS], b[U][MMA_MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + 32 * u;
      const bool in = k < K;
#pragma unroll
      for (int ns = 0; ns < NS; ++ns)
        a[u][ns].u = (in && wr[ns]) ? *reinterpret_cast<const uint4*>(wr[ns] + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int mt = 0; mt < MMA_MT; ++mt)
        b[u][mt].u = (in && mt < row_blocks && xr[mt]) ? *reinterpret_cast<const uint4*>(xr[mt] + k)
                                                       : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int mt = 0; mt < MMA_MT; ++mt) {
        if (mt < row_blocks) {
#pragma unroll
          for (int ns = 0; ns < NS; ++ns)
            acc[mt][ns] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][ns].v, b[u][mt].v, acc[mt][ns], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int mt = 0; mt < MMA_MT; ++mt) {
    const int m = 16 * mt + col;
    if (m >= rows) continue;
#pragma unroll
    for (int ns = 0; ns < NS; ++ns) {
      const int n = n_base + 16 * ns + 4 * grp;
      if (act >= MOE_ACT_GATED) {                       // a lane's four columns are two (gate, up) pairs
        bf16_t* o = out + (size_t)(first + m) * (N / 2) + n / 2;
#pragma unroll
        for (int i = 0; i < 4; i += 2)
          if (n + i + 1 < N) o[i / 2] = float_to_bf16(moe_gated(acc[mt][ns][i], acc[mt][ns][i + 1], act));
        continue;
      }
      bf16_t* o = out + (size_t)(first + m) * N + n;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (n + i < N) {
          const float v = acc[mt][ns][i];
          o[i] = float_to_bf16(act >= 0 ? moe_gelu(v, act) : v);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The product for experts with many rows (prompts): tiles of 128 slots by 128 columns, x and W
// through shared memory in slices of 64 k, two stages (the next slice is read from memory while
// the current one is multiplied, and written to the other stage behind one barrier a slice). The
// four wavefronts own 128 x 32 each: per half slice up to eight operands of x and two of W from
// shared memory (16 bytes a lane; rows padded by 16 bytes, which spreads a read over all banks)
// for up to sixteen matrix instructions. Every sum is formed in the same order as in the kernel above.
// ---------------------------------------------------------------------------
#define BIG_TM 128
#define BIG_BN 128
#define BIG_BK 64
#define BIG_LD 72   // halfwords per row of a slice: 64 and 8 of padding

__global__ __launch_bounds__(256) void moe_linear_big_kernel(
    const bf16_t* __restrict__ x, const int* __restrict__ pair_of_slot, int gather, int pairs_per_row,
    const bf16_t* __restrict__ w, bf16_t* __restrict__ out, const int* __restrict__ tile_expert,
    const int* __restrict__ tile_first, const int* __restrict__ offsets, const int* __restrict__ n_tiles, int N, int K,
    int act) {
  extern __shared__ __align__(16) unsigned char big_smem[];
  bf16_t* xs = reinterpret_cast<bf16_t*>(big_smem);              // [2][BIG_TM * BIG_LD]
  bf16_t* ws = xs + 2 * BIG_TM * BIG_LD;                          // [2][BIG_BN * BIG_LD]
  const int tile = blockIdx.x;
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile];
  const int first = tile_first[tile];
  const int rows = min(BIG_TM, offsets[e + 1] - first);
  const int n0 = blockIdx.y * BIG_BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  // what this thread brings in per slice: four pieces of x and four of W (rows r, r + 32, ..., 16 bytes at 8 c)
  const int r = threadIdx.x >> 3, c = threadIdx.x & 7;
  const bf16_t* xsrc[4];
  const bf16_t* wsrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = r + 32 * i;
    xsrc[i] = nullptr;
    if (m < rows) {
      const int src = gather ? pair_of_slot[first + m] / pairs_per_row : first + m;
      xsrc[i] = x + (size_t)src * K + 8 * c;
    }
    const int n = n0 + r + 32 * i;
    wsrc[i] = n < N ? w + ((size_t)e * N + n) * K + 8 * c : nullptr;
  }
  uint4 px[4], pw[4];
  auto fetch = [&](int k0) {
    const bool in = k0 + 8 * c < K;              // K is a multiple of 32: the last slice may be half a slice
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      px[i] = (in && xsrc[i]) ? *reinterpret_cast<const uint4*>(xsrc[i] + k0) : make_uint4(0, 0, 0, 0);
      pw[i] = (in && wsrc[i]) ? *reinterpret_cast<const uint4*>(wsrc[i] + k0) : make_uint4(0, 0, 0, 0);
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<uint4*>(xs + stage * BIG_TM * BIG_LD + (r + 32 * i) * BIG_LD + 8 * c) = px[i];
      *reinterpret_cast<uint4*>(ws + stage * BIG_BN * BIG_LD + (r + 32 * i) * BIG_LD + 8 * c) = pw[i];
    }
  };
  // a wavefront owns all 128 rows and 32 of the columns: a tile with fewer rows then costs every
  // wavefront less (an expert's last tile holds what is left of its rows), none of them idles
  moe_f32x4_t acc[8][2];
#pragma unroll
  for (int mt = 0; mt < 8; ++mt)
#pragma unroll
    for (int ns = 0; ns < 2; ++ns) acc[mt][ns] = moe_f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int row_blocks = (rows + 15) >> 4;
  fetch(0);
  stash(0);
  __syncthreads();
  int stage = 0;
  for (int k0 = 0; k0 < K; k0 += BIG_BK) {
    const bool more = k0 + BIG_BK < K;
    if (more) fetch(k0 + BIG_BK);
    const bf16_t* xt = xs + stage * BIG_TM * BIG_LD;
    const bf16_t* wt = ws + stage * BIG_BN * BIG_LD;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      MoePack a[2], b[8];
#pragma unroll
      for (int ns = 0; ns < 2; ++ns)
        a[ns].u = *reinterpret_cast<const uint4*>(wt + (32 * wave + 16 * ns + col) * BIG_LD + 32 * half + 8 * grp);
#pragma unroll
      for (int mt = 0; mt < 8; ++mt)
        if (mt < row_blocks) b[mt].u = *reinterpret_cast<const uint4*>(xt + (16 * mt + col) * BIG_LD + 32 * half + 8 * grp);
#pragma unroll
      for (int mt = 0; mt < 8; ++mt) {
        if (mt < row_blocks) {
#pragma unroll
          for (int ns = 0; ns < 2; ++ns)
            acc[mt][ns] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ns].v, b[mt].v, acc[mt][ns], 0, 0, 0);
        }
      }
    }
    if (more) stash(stage ^ 1);
    __syncthreads();
    stage ^= 1;
  }
#pragma unroll
  for (int mt = 0; mt < 8; ++mt) {
    const int m = 16 * mt + col;
    if (m >= rows) continue;
#pragma unroll
    for (int ns = 0; ns < 2; ++ns) {
      const int n = n0 + 32 * wave + 16 * ns + 4 * grp;
      if (act >= MOE_ACT_GATED) {
        bf16_t* g = out + (size_t)(first + m) * (N / 2) + n / 2;
#pragma unroll
        for (int i = 0; i < 4; i += 2)
          if (n + i + 1 < N) g[i / 2] = float_to_bf16(moe_gated(acc[mt][ns][i], acc[mt][ns][i + 1], act));
        continue;
      }
      bf16_t* o = out + (size_t)(first + m) * N + n;
      if (n + 3 < N && (N & 3) == 0) {
        union {
          uint2 u;
          bf16_t e[4];
        } pk;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float v = acc[mt][ns][i];
          pk.e[i] = float_to_bf16(act >= 0 ? moe_gelu(v, act) : v);
        }
        *reinterpret_cast<uint2*>(o) = pk.u;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (n + i < N) {
            const float v = acc[mt][ns][i];
            o[i] = float_to_bf16(act >= 0 ? moe_gelu(v, act) : v);
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The same product with the dense path's machinery (gemm_tiles.h): K a multiple of 64; tiles of
// 128 sorted rows by 128 columns; slices of 64 k travel from memory into shared memory by loads
// that write it directly, three slices ahead of the one that is multiplied (four stages), their
// 16-byte pieces placed by the same XOR, so that operand reads meet no bank conflict; four
// wavefronts of 64 x 64. What differs from the dense kernel is where a tile's rows come from:
// the tile's expert gives the weight, its rows of x are gathered by index (a row beyond the
// tile's count reads the tile's last row and is never written).
// ---------------------------------------------------------------------------
#define GT_BM 256
#define GT_BN 128
#define GT_WM 4
#define GT_STAGES 3

__global__ __launch_bounds__(64 * GT_WM * 2) void moe_linear_tiles_kernel(
    const bf16_t* __restrict__ x, const int* __restrict__ pair_of_slot, int gather, int pairs_per_row,
    const bf16_t* __restrict__ w, bf16_t* __restrict__ out, const int* __restrict__ tile_expert,
    const int* __restrict__ tile_first, const int* __restrict__ offsets, const int* __restrict__ n_tiles, int N, int K,
    int act) {
  using namespace tiles;
  typedef Shape<GT_BM, GT_BN, GT_WM, 2, GT_STAGES> S;
  extern __shared__ __attribute__((aligned(16))) unsigned char gt_smem[];
  const int tile = blockIdx.x;
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile];
  const int first_row = tile_first[tile];
  const int rows = min(GT_BM, offsets[e + 1] - first_row);
  const int n0 = blockIdx.y * GT_BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int wm = wave % GT_WM, wn = wave / GT_WM;
  const int piece = (tid & 7) ^ ((tid >> 4) & 7);
  const bf16_t* x_src[S::X_TURNS];
  const bf16_t* w_src[S::W_TURNS];
#pragma unroll
  for (int j = 0; j < S::X_TURNS; ++j) {
    const int slot = first_row + min(S::TURN_ROWS * j + (tid >> 3), rows - 1);
    const int src = gather ? pair_of_slot[slot] / pairs_per_row : slot;
    x_src[j] = x + (size_t)src * K + 8 * piece;
  }
  const bf16_t* we = w + (size_t)e * N * K;
#pragma unroll
  for (int j = 0; j < S::W_TURNS; ++j)
    w_src[j] = we + (size_t)min(n0 + S::TURN_ROWS * j + (tid >> 3), N - 1) * K + 8 * piece;
  typedef __attribute__((address_space(3))) unsigned char* lds_ptr;
  const unsigned smem_lds = (unsigned)(unsigned long)(lds_ptr)gt_smem;
  auto load_to_lds = [&](const void* src, unsigned lds) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds) : "memory", "m0");
  };
  auto copy_step = [&](int kt, int stage) {
    const unsigned base = __builtin_amdgcn_readfirstlane(smem_lds + stage * S::STAGE_BYTES + 1024 * wave);
#pragma unroll
    for (int j = 0; j < S::X_TURNS; ++j) load_to_lds(x_src[j] + (size_t)kt * BK, base + 16 * S::THREADS * j);
#pragma unroll
    for (int j = 0; j < S::W_TURNS; ++j)
      load_to_lds(w_src[j] + (size_t)kt * BK, base + GT_BM * ROW_BYTES + 16 * S::THREADS * j);
  };
  // loads complete in the order they were issued: with no more than the later steps' loads
  // outstanding, this thread's share of the next step has landed
  auto wait_for_step = [&](int steps_after) {
    if (steps_after <= 0)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S::LOADS) : "memory");
  };
  static_assert(GT_STAGES == 3 && S::LOADS < 64, "the wait counts above");
  const int swz = (col >> 1) & 7;
  int read_off[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) read_off[s] = col * ROW_BYTES + 16 * ((4 * s + grp) ^ swz);
  const int x_half = wm * (GT_BM / GT_WM) * ROW_BYTES, w_half = GT_BM * ROW_BYTES + wn * (GT_BN / 2) * ROW_BYTES;
  f32x4_t acc[S::MI][S::NJ];
#pragma unroll
  for (int i = 0; i < S::MI; ++i)
#pragma unroll
    for (int j = 0; j < S::NJ; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int row_blocks = min(S::MI, max(0, (rows - wm * (GT_BM / GT_WM) + 15) >> 4));   // of this wavefront's 64 rows
  const int steps = K / BK;
#pragma unroll
  for (int ahead = 0; ahead < GT_STAGES - 1; ++ahead)
    if (ahead < steps) copy_step(ahead, ahead);
  for (int kt = 0; kt < steps; ++kt) {
    wait_for_step(min(kt + GT_STAGES - 2, steps - 1) - kt);
    __syncthreads();
    if (kt + GT_STAGES - 1 < steps) copy_step(kt + GT_STAGES - 1, (kt + GT_STAGES - 1) % GT_STAGES);
    const unsigned char* st = gt_smem + (kt % GT_STAGES) * S::STAGE_BYTES;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      Frag xf[S::MI], wf[S::NJ];
#pragma unroll
      for (int i = 0; i < S::MI; ++i)
        xf[i].u = *reinterpret_cast<const uint4*>(st + x_half + 16 * i * ROW_BYTES + read_off[s]);
#pragma unroll
      for (int j = 0; j < S::NJ; ++j)
        wf[j].u = *reinterpret_cast<const uint4*>(st + w_half + 16 * j * ROW_BYTES + read_off[s]);
#pragma unroll
      for (int i = 0; i < S::MI; ++i) {
        if (i < row_blocks) {
#pragma unroll
          for (int j = 0; j < S::NJ; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j].v, xf[i].v, acc[i][j], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < S::MI; ++i) {
    const int m = wm * (GT_BM / GT_WM) + 16 * i + col;
    if (m >= rows) continue;
#pragma unroll
    for (int j = 0; j < S::NJ; ++j) {
      const int n = n0 + wn * (GT_BN / 2) + 16 * j + 4 * grp;
      if (n >= N) continue;
      f32x4_t c = acc[i][j];
      if (act >= MOE_ACT_GATED) {
        bf16_t* g = out + (size_t)(first_row + m) * (N / 2) + n / 2;
#pragma unroll
        for (int q = 0; q < 4; q += 2)
          if (n + q + 1 < N) g[q / 2] = float_to_bf16(moe_gated(c[q], c[q + 1], act));
        continue;
      }
      if (act >= 0) {
#pragma unroll
        for (int q = 0; q < 4; ++q) c[q] = moe_gelu(c[q], act);
      }
      bf16_t* o = out + (size_t)(first_row + m) * N + n;
      if (n + 3 < N && (N % 4) == 0) {
        *reinterpret_cast<uint2*>(o) = pack_bf16x4(c);
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (n + q < N) o[q] = float_to_bf16(c[q]);
      }
    }
  }
}

// out[t, :] = sum_k weights[t, k] * y[slot_of_pair[t * top + k], :] (+ shared[t, :]), float32 sums in
// the order k = 0, 1, ..., the shared expert last; rounded once. Without `weights` every weight is 1
// (experts whose inputs carried the weight). With `shared_gate` (one float32 logit per token, the
// tokens' `gate_stride` apart) the shared row is multiplied by sigmoid(shared_gate[t]).
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ slot_of_pair,
                                   const float* __restrict__ weights, const T* __restrict__ shared,
                                   const float* __restrict__ shared_gate, long gate_stride,
                                   T* __restrict__ out, int width, int top) {
  __shared__ int slots[64];
  __shared__ float share[64];
  const int t = blockIdx.x;
  const int kept = min(top, 64);           // a token's first choices wait in shared memory, so that the rows' loads do not wait for them one by one
  if ((int)threadIdx.x < kept) {
    slots[threadIdx.x] = slot_of_pair[(size_t)t * top + threadIdx.x];
    share[threadIdx.x] = weights ? weights[(size_t)t * top + threadIdx.x] : 1.f;
  }
  __syncthreads();
  const int j = blockIdx.y * blockDim.x + threadIdx.x;
  if (j >= width) return;
  float acc = 0.f;
  for (int k = 0; k < kept; ++k) acc += share[k] * to_float(y[(size_t)slots[k] * width + j]);
  for (int k = kept; k < top; ++k)
    acc += (weights ? weights[(size_t)t * top + k] : 1.f) * to_float(y[(size_t)slot_of_pair[(size_t)t * top + k] * width + j]);
  if (shared) {
    const float open = shared_gate ? 1.f / (1.f + expf(-shared_gate[(size_t)t * gate_stride])) : 1.f;
    acc += open * to_float(shared[(size_t)t * width + j]);
  }
  out[(size_t)t * width + j] = from_float<T>(acc);
}

extern "C" int q3_moe_pick(const float* logits, long row_stride, int n_tokens, int E, int top, int mode,
                           const float* correction, int groups, int keep, int* chosen, float* weights,
                           hipStream_t stream) {
  if (n_tokens <= 0 || E <= 0 || top <= 0 || top > E || E > 4096 || mode < 0 || mode > 2 || row_stride < E)
    return Q3_ERR_BAD_ARGUMENT;
  if (mode != 2) groups = keep = 1;
  if (mode == 2 && (!correction || groups <= 0 || E % groups || keep <= 0 || keep > groups || top > keep * (E / groups)))
    return Q3_ERR_BAD_ARGUMENT;
  const int waves = 4;
  const size_t smem = (size_t)waves * (E + top + groups) * sizeof(float);
  hipLaunchKernelGGL(moe_pick_kernel, dim3((n_tokens + waves - 1) / waves), dim3(waves * Q3_WAVE), smem, stream, logits,
                     row_stride, n_tokens, E, top, mode, correction, groups, keep, chosen, weights);
  return q3_launch_status();
}

// Slots per tile: 16 for the float32 multiply-add kernel, 64 for the matrix-core kernel, 128 for
// its form for experts with many rows, 256 for that with inner sizes in steps of 64 (`matrix_cores` 0, 1, 2, 3).
extern "C" int q3_moe_tile_rows(int matrix_cores) {
  return matrix_cores == 3 ? GT_BM : matrix_cores == 2 ? BIG_TM : matrix_cores ? MMA_TM : MOE_BM;
}

extern "C" int q3_moe_align(const int* chosen, int P, int E, int tile_rows, int* offsets, int* pair_of_slot,
                            int* slot_of_pair, int* tile_expert, int* tile_first, int* n_tiles, hipStream_t stream) {
  if (P <= 0 || E <= 0 || E > 4096 ||
      (tile_rows != MOE_BM && tile_rows != MMA_TM && tile_rows != BIG_TM && tile_rows != GT_BM))
    return Q3_ERR_BAD_ARGUMENT;
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (size_t)2 * E * sizeof(int), stream, chosen, P, E,
                     tile_rows, offsets, pair_of_slot, slot_of_pair, tile_expert, tile_first, n_tiles);
  return q3_launch_status();
}

// The matrix-core product: bfloat16, K a multiple of 32, tiles of 64 slots.
extern "C" int q3_moe_linear_mma(const void* x, const int* pair_of_slot, int gather, int pairs_per_row, const void* w,
                                 void* out, const int* tile_expert, const int* tile_first, const int* offsets,
                                 const int* n_tiles, int max_tiles, int N, int K, int act, int tile_rows,
                                 hipStream_t stream) {
  if (max_tiles <= 0 || N <= 0 || K <= 0 || K % 32 || pairs_per_row <= 0 || act < -1 || act > MOE_ACT_MOST ||
      (act >= MOE_ACT_GATED && N % 2) ||
      (tile_rows != MMA_TM && tile_rows != BIG_TM && tile_rows != GT_BM))
    return Q3_ERR_BAD_ARGUMENT;
  if (tile_rows == GT_BM) {         // the dense path's copies and stages
    typedef tiles::Shape<GT_BM, GT_BN, GT_WM, 2, GT_STAGES> S;
    const dim3 grid(max_tiles, (N + GT_BN - 1) / GT_BN);
    if (grid.y > 65535 || K % 64) return Q3_ERR_UNSUPPORTED;
    hipError_t attr = hipFuncSetAttribute((const void*)moe_linear_tiles_kernel,
                                          hipFuncAttributeMaxDynamicSharedMemorySize, S::SMEM_BYTES);
    if (attr != hipSuccess) return (int)attr;
    hipLaunchKernelGGL(moe_linear_tiles_kernel, grid, dim3(S::THREADS), S::SMEM_BYTES, stream, (const bf16_t*)x,
                       pair_of_slot, gather, pairs_per_row, (const bf16_t*)w, (bf16_t*)out, tile_expert, tile_first,
                       offsets, n_tiles, N, K, act);
    return q3_launch_status();
  }
  if (tile_rows == BIG_TM) {
    const dim3 big(max_tiles, (N + BIG_BN - 1) / BIG_BN);
    if (big.y > 65535) return Q3_ERR_UNSUPPORTED;
    const size_t smem = (size_t)2 * (BIG_TM + BIG_BN) * BIG_LD * sizeof(bf16_t);
    hipError_t attr = hipFuncSetAttribute((const void*)moe_linear_big_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)smem);
    if (attr != hipSuccess) return (int)attr;
    hipLaunchKernelGGL(moe_linear_big_kernel, big, dim3(256), smem, stream, (const bf16_t*)x, pair_of_slot, gather,
                       pairs_per_row, (const bf16_t*)w, (bf16_t*)out, tile_expert, tile_first, offsets, n_tiles, N, K, act);
    return q3_launch_status();
  }
  // few blocks (steps of few tokens): one slab of 16 columns per wavefront, so that more blocks stream the weights
  const bool narrow = (long)max_tiles * ((N + 255) / 256) < 512;
  const int per_block = narrow ? 64 : 256;
  const dim3 grid(max_tiles, (N + per_block - 1) / per_block);
  if (grid.y > 65535) return Q3_ERR_UNSUPPORTED;
  if (narrow)
    hipLaunchKernelGGL(moe_linear_mma_kernel<1>, grid, dim3(256), 0, stream, (const bf16_t*)x, pair_of_slot, gather,
                       pairs_per_row, (const bf16_t*)w, (bf16_t*)out, tile_expert, tile_first, offsets, n_tiles, N, K, act);
  else
    hipLaunchKernelGGL(moe_linear_mma_kernel<4>, grid, dim3(256), 0, stream, (const bf16_t*)x, pair_of_slot, gather,
                       pairs_per_row, (const bf16_t*)w, (bf16_t*)out, tile_expert, tile_first, offsets, n_tiles, N, K, act);
  return q3_launch_status();
}

extern "C" int q3_moe_linear(const void* x, const int* pair_of_slot, int gather, int pairs_per_row, const void* w,
                             void* out, const int* tile_expert, const int* tile_first, const int* offsets,
                             const int* n_tiles, int max_tiles, int N, int K, int act, int dtype,
                             hipStream_t stream) {
  if (max_tiles <= 0 || N <= 0 || K <= 0 || pairs_per_row <= 0 || act < -1 || act > MOE_ACT_MOST ||
      (act >= MOE_ACT_GATED && N % 2))
    return Q3_ERR_BAD_ARGUMENT;
  const dim3 grid(max_tiles, (N + MOE_BN - 1) / MOE_BN);
  if (grid.y > 65535) return Q3_ERR_UNSUPPORTED;
  Q3_DISPATCH_DTYPE(dtype, TT,
                    hipLaunchKernelGGL(moe_linear_kernel<TT>, grid, dim3(256), 0, stream, (const TT*)x, pair_of_slot,
                                       gather, pairs_per_row, (const TT*)w, (TT*)out, tile_expert, tile_first, offsets,
                                       n_tiles, N, K, act));
  return q3_launch_status();
}

extern "C" int q3_moe_combine(const void* y, const int* slot_of_pair, const float* weights, const void* shared,
                              const float* shared_gate, long gate_stride, void* out, int n_tokens, int width, int top,
                              int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || width <= 0 || top <= 0 || (shared_gate && !shared)) return Q3_ERR_BAD_ARGUMENT;
  int threads = 64;
  while (threads < 256 && threads < width) threads *= 2;
  if ((width + threads - 1) / threads > 65535) return Q3_ERR_UNSUPPORTED;
  Q3_DISPATCH_DTYPE(dtype, TT,
                    hipLaunchKernelGGL(moe_combine_kernel<TT>, dim3(n_tokens, (width + threads - 1) / threads),
                                       dim3(threads), 0, stream, (const TT*)y,
                                       slot_of_pair, weights, (const TT*)shared, shared_gate, gate_stride, (TT*)out,
                                       width, top));
  return q3_launch_status();
}
