// Latent attention: queries, keys and values that pass through narrow normalised vectors, of
// which only the key/value latent and one rotated key part shared by all heads are cached.
//
// The cache holds one row of Dk = kv_rank + rot_dim numbers per token: [c | k_rot], c the
// normalised latent, k_rot the rotated part. Attention runs in the latent's space: with
// k_h = U_h c (the per-head key made from the latent) a score is
//   q_h . k_h + q_rot . k_rot = (U_h^T q_h) . c + q_rot . k_rot,
// so a query row becomes [U_h^T q_h | q_rot] (Dk numbers) and every head reads the same cached
// rows as keys; the softmax-weighted sum of the rows' first kv_rank numbers is then multiplied by
// the head's value matrix. Scores, softmax statistics, weights and sums are float32.
#include "common.h"

#include <math.h>

// ---------------------------------------------------------------------------
// One block per token. `down` (T, q_rank + kv_rank + rot_dim) is the joint down-projection; its rows
// lie `down_stride` numbers apart (a wider product may carry further columns behind these), and
// rot_dim may be 0 (keys without a rotated part).
//   cq[t]    = rms_norm(down[t, :q_rank]) * q_weight                       -> (T, q_rank)
//   cache row of (sequence, position) = [rms_norm(down[t, q_rank:q_rank+kv_rank]) * kv_weight |
//                                        rotate(down[t, q_rank+kv_rank:])]
// The rotation turns pairs (2i, 2i+1), i < rot_pairs, by angle = float(position) * inv_freq[i]
// (a float32 product), with cos and sin multiplied by rot_factor; numbers beyond 2 rot_pairs pass.
// ---------------------------------------------------------------------------
template <typename T, typename W>
__global__ void latent_prepare_kernel(const T* __restrict__ down, long down_stride, int q_rank, int kv_rank, int rot_dim,
                                      const W* __restrict__ q_weight, const W* __restrict__ kv_weight, float eps,
                                      const float* __restrict__ inv_freq, int rot_pairs, float rot_factor,
                                      const int* __restrict__ positions, const int* __restrict__ seq_index,
                                      const int* __restrict__ block_table, int bt_stride, int bt_rows,
                                      T* __restrict__ cache, int page, int num_pages, T* __restrict__ cq) {
  extern __shared__ float smem[];
  float* red = smem;
  float* row = smem + 32;
  const int t = blockIdx.x;
  const int R = q_rank + kv_rank + rot_dim;
  const T* src = down + (size_t)t * down_stride;
  float acc_q = 0.f, acc_kv = 0.f;
  for (int j = threadIdx.x; j < R; j += blockDim.x) {
    const float v = to_float(src[j]);
    row[j] = v;
    if (j < q_rank) acc_q += v * v;
    else if (j < q_rank + kv_rank) acc_kv += v * v;
  }
  const float q_scale = rsqrtf(block_sum(acc_q, red) / (float)q_rank + eps);
  const float kv_scale = rsqrtf(block_sum(acc_kv, red) / (float)kv_rank + eps);
  for (int j = threadIdx.x; j < q_rank; j += blockDim.x)
    cq[(size_t)t * q_rank + j] = from_float<T>(row[j] * q_scale * to_float(q_weight[j]));
  if (!cache) return;
  const int pos = positions[t];
  const int seq = seq_index[t];
  if (seq < 0 || seq >= bt_rows || pos < 0 || pos / page >= bt_stride) return;
  const int pg = block_table[(size_t)seq * bt_stride + pos / page];
  if (pg < 0 || pg >= num_pages) return;
  T* dst = cache + ((size_t)pg * page + pos % page) * (kv_rank + rot_dim);
  const float* kv = row + q_rank;
  for (int j = threadIdx.x; j < kv_rank; j += blockDim.x)
    dst[j] = from_float<T>(kv[j] * kv_scale * to_float(kv_weight[j]));
  const float* tail = kv + kv_rank;
  for (int i = threadIdx.x; i < rot_pairs; i += blockDim.x) {
    const float a = (float)pos * inv_freq[i];
    const float c = cosf(a) * rot_factor, s = sinf(a) * rot_factor;
    const float u = tail[2 * i], v = tail[2 * i + 1];
    dst[kv_rank + 2 * i] = from_float<T>(u * c - v * s);
    dst[kv_rank + 2 * i + 1] = from_float<T>(v * c + u * s);
  }
  for (int j = 2 * rot_pairs + threadIdx.x; j < rot_dim; j += blockDim.x) dst[kv_rank + j] = from_float<T>(tail[j]);
}

// ---------------------------------------------------------------------------
// y[t, h, :] = W[h] x[t, h, :] for every head: x rows of `I` numbers at x + t * x_row + h * x_head,
// W (H, O, I) row-major (a result's weights side by side), y rows of `O` numbers at
// out + t * out_row + h * out_head. The general kernel: one block is 16 tokens of one head and up
// to 256 output columns; the tokens' inputs wait in shared memory, each thread owns one output
// column and walks I in order with float32 sums.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void headwise_linear_kernel(const T* __restrict__ x, long x_row, int x_head,
                                                              const T* __restrict__ w, T* __restrict__ out,
                                                              long out_row, int out_head, int n_rows, int I, int O) {
  extern __shared__ float xs[];  // [16][I]
  const int m0 = blockIdx.x * 16;
  const int h = blockIdx.y;
  const int rows = min(16, n_rows - m0);
  for (int idx = threadIdx.x; idx < 16 * I; idx += blockDim.x) {
    const int m = idx / I, i = idx - m * I;
    xs[idx] = m < rows ? to_float(x[(size_t)(m0 + m) * x_row + (size_t)h * x_head + i]) : 0.f;
  }
  __syncthreads();
  const int o = blockIdx.z * blockDim.x + threadIdx.x;
  if (o >= O) return;
  float acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = 0.f;
  const T* wh = w + ((size_t)h * O + o) * I;
  for (int i = 0; i < I; ++i) {
    const float wv = to_float(wh[i]);
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] += xs[m * I + i] * wv;
  }
  for (int m = 0; m < rows; ++m)
    out[(size_t)(m0 + m) * out_row + (size_t)h * out_head + o] = from_float<T>(acc[m]);
}

// The same on the matrix cores (v_mfma_f32_16x16x32_bf16): bfloat16, I a multiple of 32, rows of x
// that start at multiples of 16 bytes. y^T (columns x tokens) = W_h (columns x I) . x_h^T: 16 weight
// rows are the first operand, 16 tokens' rows the second, both straight from memory. A wavefront
// owns 16 MT tokens and 128 output columns of one head (8 slabs of 16): per step of 32 k it reads
// MT operands of x and 8 of W for 8 MT matrix instructions.
typedef __attribute__((ext_vector_type(8))) __bf16 lat_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float lat_f32x4_t;
union LatPack {
  uint4 u;
  uint2 h[2];
  lat_bf16x8_t v;
  __bf16 e[8];
};

template <int MT>
__global__ __launch_bounds__(256) void headwise_linear_mma_kernel(const bf16_t* __restrict__ x, long x_row, int x_head,
                                                                  const bf16_t* __restrict__ w,
                                                                  bf16_t* __restrict__ out, long out_row, int out_head,
                                                                  int n_rows, int I, int O) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int h = blockIdx.y;
  const int t0 = (blockIdx.x * 4 + wave) * 16 * MT;
  if (t0 >= n_rows) return;
  const int o_base = blockIdx.z * 128;
  const bf16_t* xr[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int t = t0 + 16 * mt + col;
    xr[mt] = t < n_rows ? x + (size_t)t * x_row + (size_t)h * x_head + 8 * grp : nullptr;
  }
  const bf16_t* wr[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const int o = o_base + 16 * s + col;
    wr[s] = o < O ? w + ((size_t)h * O + o) * I + 8 * grp : nullptr;
  }
  lat_f32x4_t acc[MT][8];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int s = 0; s < 8; ++s) acc[mt][s] = lat_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int k0 = 0; k0 < I; k0 += 32) {
    LatPack a[8], b[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      b[mt].u = xr[mt] ? *reinterpret_cast<const uint4*>(xr[mt] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int s = 0; s < 8; ++s) a[s].u = wr[s] ? *reinterpret_cast<const uint4*>(wr[s] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt][s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s].v, b[mt].v, acc[mt][s], 0, 0, 0);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int t = t0 + 16 * mt + col;
    if (t >= n_rows) continue;
    bf16_t* o_row = out + (size_t)t * out_row + (size_t)h * out_head;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int o = o_base + 16 * s + 4 * grp;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (o + i < O) o_row[o + i] = float_to_bf16(acc[mt][s][i]);
    }
  }
}

// The rotated tail of every query head: out[t, h, j] = rotate(x[t, h, j]) for the `rot_dim`
// numbers at x + t * x_row + h * x_head (+ j), written at out + t * out_row + h * out_head.
template <typename T>
__global__ void rotate_heads_kernel(const T* __restrict__ x, long x_row, int x_head, T* __restrict__ out,
                                    long out_row, int out_head, int H, int rot_dim, int rot_pairs,
                                    const float* __restrict__ inv_freq, float rot_factor,
                                    const int* __restrict__ positions) {
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = (rot_dim + 1) / 2;       // work items per head: a pair, or a number that passes
  for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
    const int h = idx / half, i = idx - h * half;
    const T* src = x + (size_t)t * x_row + (size_t)h * x_head;
    T* dst = out + (size_t)t * out_row + (size_t)h * out_head;
    if (i < rot_pairs) {
      const float a = pos * inv_freq[i];
      const float c = cosf(a) * rot_factor, s = sinf(a) * rot_factor;
      const float u = to_float(src[2 * i]), v = to_float(src[2 * i + 1]);
      dst[2 * i] = from_float<T>(u * c - v * s);
      dst[2 * i + 1] = from_float<T>(v * c + u * s);
    } else {
      dst[2 * i] = src[2 * i];
      if (2 * i + 1 < rot_dim) dst[2 * i + 1] = src[2 * i + 1];
    }
  }
}

// ---------------------------------------------------------------------------
// The general attention kernel: any sizes, float32 or bfloat16 storage, float32 arithmetic.
// A sequence's query rows are numbered (token, head), head fastest; a block serves 16 consecutive
// rows against tiles of 32 cached rows, which are keys (all Dk numbers) and values (the first Dv)
// at once, so a tile is loaded once. Tiles start at absolute positions that are multiples of 32,
// so the order in which a row's sums are formed does not depend on how the sequence was cut into
// steps or on what else the block serves. Row of token i (position p = kv_len - q_len + i) sees
// positions j <= p, and with a window w > 0 only p - j < w. With `sink` (H floats) the softmax's
// denominator of head h also holds exp(sink[h]), a term without a key and a value that is not
// scaled; with `gate` (rows `gate_stride` apart, H numbers each) head h's result is multiplied by
// sigmoid(gate[token, h]).
// ---------------------------------------------------------------------------
#define LAT_BM 16
#define LAT_BN 32

template <typename T, int NV>
__global__ __launch_bounds__(256) void latent_attn_kernel(const T* __restrict__ q, T* __restrict__ out,
                                                          const T* __restrict__ cache, int num_pages,
                                                          const int* __restrict__ block_table, int bt_stride,
                                                          const int* __restrict__ cu_q,
                                                          const int* __restrict__ kv_lens, int H, int Dk, int Dv,
                                                          int page, float scale, int window,
                                                          const float* __restrict__ sink, const T* __restrict__ gate,
                                                          long gate_stride) {
  extern __shared__ float smem[];
  const int b = blockIdx.y;
  const int q0 = cu_q[b];
  const int q_len = cu_q[b + 1] - q0;
  const int n_rows = q_len * H;
  const int m0 = blockIdx.x * LAT_BM;
  if (m0 >= n_rows) return;
  const int rows = min(LAT_BM, n_rows - m0);
  const int kv_len = kv_lens[b];
  const int base_pos = kv_len - q_len;
  const int ldk = Dk + 1;
  float* qs = smem;                    // [BM][Dk]
  float* kv = qs + LAT_BM * Dk;        // [BN][Dk + 1]
  float* ps = kv + LAT_BN * ldk;       // [BM][BN + 1]
  const int t = threadIdx.x;
  const int r = t >> 4;
  const int sub = t & 15;
  const bool my_row = r < rows;
  const int my_tok = (m0 + (my_row ? r : 0)) / H;
  const int my_head = (m0 + (my_row ? r : 0)) - my_tok * H;
  const int my_pos = base_pos + my_tok;

  for (int idx = t; idx < LAT_BM * Dk; idx += 256) {
    const int rr = idx / Dk, d = idx - rr * Dk;
    float v = 0.f;
    if (rr < rows) {
      const int R = m0 + rr;
      v = to_float(q[((size_t)(q0 + R / H) * H + R % H) * Dk + d]);
    }
    qs[idx] = v;
  }
  float acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const int first_tok = m0 / H, last_tok = (m0 + rows - 1) / H;
  const int k_end = base_pos + last_tok + 1;
  int k_begin = window > 0 ? max(0, base_pos + first_tok - window + 1) : 0;
  k_begin -= k_begin % LAT_BN;

  for (int kt = k_begin; kt < k_end; kt += LAT_BN) {
    __syncthreads();
    for (int jj = r; jj < LAT_BN; jj += 16) {
      const int kj = kt + jj;
      const T* src = nullptr;
      if (kj < k_end) {
        const int pg = block_table[(size_t)b * bt_stride + kj / page];
        if (pg >= 0 && pg < num_pages) src = cache + ((size_t)pg * page + kj % page) * Dk;
      }
      for (int d = sub; d < Dk; d += 16) kv[jj * ldk + d] = src ? to_float(src[d]) : 0.f;
    }
    __syncthreads();
    float s[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int jj = sub + 16 * u;
      const int kj = kt + jj;
      float dot = 0.f;
      for (int d = 0; d < Dk; ++d) dot += qs[r * Dk + d] * kv[jj * ldk + d];
      bool seen = my_row && kj <= my_pos;
      if (window > 0 && my_pos - kj >= window) seen = false;
      s[u] = seen ? dot * scale : -INFINITY;
    }
    float tile_max = fmaxf(s[0], s[1]);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, off, Q3_WAVE));
    const float m_new = fmaxf(m_run, tile_max);
    float alpha = 1.f, p[2] = {0.f, 0.f};
    if (m_new > -INFINITY) {
      alpha = expf(m_run - m_new);
      p[0] = expf(s[0] - m_new);
      p[1] = expf(s[1] - m_new);
    }
    float tile_sum = p[0] + p[1];
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) tile_sum += __shfl_xor(tile_sum, off, Q3_WAVE);
    l_run = l_run * alpha + tile_sum;
    m_run = m_new;
    ps[r * (LAT_BN + 1) + sub] = p[0];
    ps[r * (LAT_BN + 1) + sub + 16] = p[1];
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] *= alpha;
    __syncthreads();
    for (int jj = 0; jj < LAT_BN; ++jj) {
      const float pj = ps[r * (LAT_BN + 1) + jj];
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int col = sub + 16 * i;
        if (col < Dv) acc[i] += pj * kv[jj * ldk + col];
      }
    }
  }
  if (my_row) {
    if (sink) l_run += expf(sink[my_head] - m_run);
    float inv = 1.f / l_run;
    if (gate) inv /= 1.f + expf(-to_float(gate[(size_t)(q0 + my_tok) * gate_stride + my_head]));
    T* o = out + ((size_t)(q0 + my_tok) * H + my_head) * Dv;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int col = sub + 16 * i;
      if (col < Dv) o[col] = from_float<T>(acc[i] * inv);
    }
  }
}

// ---------------------------------------------------------------------------
// The matrix-core kernel (v_mfma_f32_16x16x32_bf16): bfloat16, Dk a multiple of 32, Dv of 16.
// A block of four wavefronts serves 64 consecutive (token, head) rows of one sequence, 16 per
// wavefront, against tiles of 32 cached rows that start at absolute positions in steps of 32.
// Every tile goes from the cache to shared memory once for all 64 rows and twice over: as it is
// (keys: a lane's operand is 16 bytes of one cached row) and transposed (values: a lane's
// operand is two runs of four keys of one column), because the first product sums over a row's
// numbers and the second over the keys:
//   S^T (keys x rows)  = K (keys x Dk) . Q^T          first operand K rows, second Q rows (registers)
//   O^T (Dv x rows)   += V^T (Dv x keys) . P^T        first operand V^T rows, second P
// Both leave a query row in the lanes l, l + 16, l + 32, l + 48, so a row's statistics, weights and
// sums stay where they are. After S^T a lane holds the scores of keys 4g..4g+3 of both 16-key
// halves (g = lane / 16); the second product numbers its summed index so that these are the
// lane's eight, and the transposed copy keeps a row's keys in that order. Scores, maxima, sums and the output sums are float32;
// weights are rounded to bfloat16 as the second product's operand.
// ---------------------------------------------------------------------------
#define LMA_ROWS 64
#define LMA_BN 32
#define LMA_KPAD 8
#define LMA_VLD 40   // halfwords per transposed row: 32 keys and 8 of padding

// Which sequence and which of its row tiles a block serves: blocks are numbered through the
// sequences' tiles of 64 rows in turn (a step's sequences bring very different numbers of rows, and
// a grid of the longest's tiles for every sequence would be mostly blocks that start and end).
__device__ inline bool lma_find_tile(const int* __restrict__ cu_q, int B, int H, int tile, int& b, int& m0) {
  int at = 0;
  for (int i = 0; i < B; ++i) {
    const int n = ((cu_q[i + 1] - cu_q[i]) * H + LMA_ROWS - 1) / LMA_ROWS;
    if (tile < at + n) {
      b = i;
      m0 = (tile - at) * LMA_ROWS;
      return true;
    }
    at += n;
  }
  return false;
}

// KS: most steps of 32 over Dk; NV: most slabs of 16 over Dv that one wavefront sums; HALVES: 1, or 2
// for wide values: eight wavefronts a block, of which wavefronts w and w + 4 serve the same sixteen rows
// (both form the scores) and each sums half of the value's columns, so that a wavefront's registers
// leave room for two wavefronts a SIMD. With `splits` > 1 (blockIdx.y) a
// block walks its share of the tiles and leaves float32 sums that are not yet divided, with the
// row's maximum (in the exponent's units) and sum, in `partial` ((rows, splits, Dv + 2) floats,
// rows numbered (packed token, head)); `latent_attn_merge_kernel` joins the shares in their order.
// `sink` and `gate` as in the general kernel; with shares they join in the merge.
template <int KS, int NV, int HALVES>
__global__ __launch_bounds__(256 * HALVES) void latent_attn_mma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                                                              const bf16_t* __restrict__ cache, int num_pages,
                                                              const int* __restrict__ block_table, int bt_stride,
                                                              const int* __restrict__ cu_q,
                                                              const int* __restrict__ kv_lens, int B, int H, int Dk,
                                                              int Dv, int page, float scale_log2, int window,
                                                              int splits, float* __restrict__ partial,
                                                              const float* __restrict__ sink,
                                                              const bf16_t* __restrict__ gate, long gate_stride) {
  extern __shared__ __align__(16) unsigned char lma_smem[];
  int b, m0;
  if (!lma_find_tile(cu_q, B, H, blockIdx.x, b, m0)) return;
  const int q0 = cu_q[b];
  const int q_len = cu_q[b + 1] - q0;
  const int n_rows = q_len * H;
  const int kv_len = kv_lens[b];
  const int base_pos = kv_len - q_len;
  const int ldk = Dk + LMA_KPAD;                              // halfwords per key row
  bf16_t* kt = reinterpret_cast<bf16_t*>(lma_smem);           // [32][ldk]
  bf16_t* vt = kt + LMA_BN * ldk;                             // [Dv][LMA_VLD]
  const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3, half = threadIdx.x >> 8;
  const int col = lane & 15, grp = lane >> 4;
  const int ks = Dk >> 5;
  const int slabs = Dv >> 4, per_half = (slabs + HALVES - 1) / HALVES;
  const int nb0 = half * per_half;                            // this wavefront's first slab of the value
  const int nv = max(0, min(per_half, slabs - nb0));

  // the block's span of keys (and of that this block's share), and this wavefront's
  const int block_last = min(m0 + LMA_ROWS, n_rows) - 1;
  int k_end = base_pos + block_last / H + 1;
  int k_begin = window > 0 ? max(0, base_pos + m0 / H - window + 1) : 0;
  k_begin -= k_begin % LMA_BN;
  if (splits > 1) {
    const int tiles = (k_end - k_begin + LMA_BN - 1) / LMA_BN;
    const int share = (tiles + splits - 1) / splits;
    const int first = k_begin + blockIdx.y * share * LMA_BN;
    k_end = min(k_end, first + share * LMA_BN);
    k_begin = first;
  }
  const int w0 = m0 + 16 * wave;
  const bool wave_active = w0 < n_rows;
  const int wave_last = min(w0 + 16, n_rows) - 1;
  const int wave_k_end = wave_active ? base_pos + wave_last / H + 1 : 0;
  const int wave_k_begin = (wave_active && window > 0) ? max(0, base_pos + w0 / H - window + 1) : 0;
  const bool wave_full = wave_active && w0 + 16 <= n_rows;    // all sixteen rows are rows of the sequence
  const int wave_first_pos = base_pos + w0 / H, wave_last_pos = base_pos + wave_last / H;

  const int R = w0 + col;
  const bool valid = R < n_rows;
  const int Rc = valid ? R : (wave_active ? wave_last : 0);
  const int tok = Rc / H, head = Rc - tok * H;
  const int pos = base_pos + tok;
  LatPack qreg[KS];
  {
    const bf16_t* qr = q + ((size_t)(q0 + tok) * H + head) * Dk + 8 * grp;
#pragma unroll
    for (int i = 0; i < KS; ++i)
      qreg[i].u = (i < ks && wave_active) ? *reinterpret_cast<const uint4*>(qr + 32 * i) : make_uint4(0, 0, 0, 0);
  }
  lat_f32x4_t acc[NV];
#pragma unroll
  for (int nb = 0; nb < NV; ++nb) acc[nb] = lat_f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  // a tile's pieces on their way from the cache into registers: eight threads a key, each takes
  // every eighth piece of 16 bytes of its key's row, so that a thread looks its key's page up once
  // a tile and eight neighbours read 128 bytes in a row
  const int chunks_per_key = Dk >> 3;
  constexpr int PER_KEY = 8 * HALVES;                         // threads a key
  constexpr int NCH = (KS * 4 + PER_KEY - 1) / PER_KEY;       // pieces per thread
  const int my_key = threadIdx.x / PER_KEY, my_sub = threadIdx.x % PER_KEY;
  uint4 pre[NCH];
  // The page of a key is looked up a tile before its row is asked for, so that a tile's loads do
  // not wait for their addresses: the row's load is one trip to memory, not two in a row.
  auto lookup = [&](int kt0) -> int {
    const int kj = kt0 + my_key;
    return kj < k_end ? block_table[(size_t)b * bt_stride + kj / page] : -1;
  };
  auto fetch = [&](int kt0, int pg) {
    const int kj = kt0 + my_key;
    const bf16_t* src = (pg >= 0 && pg < num_pages) ? cache + ((size_t)pg * page + kj % page) * Dk : nullptr;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int part = my_sub + PER_KEY * i;
      pre[i] = (src && part < chunks_per_key) ? *reinterpret_cast<const uint4*>(src + 8 * part) : make_uint4(0, 0, 0, 0);
    }
  };

  int next_page = -1;
  if (k_begin < k_end) {
    fetch(k_begin, lookup(k_begin));
    next_page = lookup(k_begin + LMA_BN);
  }
  for (int kt0 = k_begin; kt0 < k_end; kt0 += LMA_BN) {
    __syncthreads();                                          // the last tile's readers are done
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int part = my_sub + PER_KEY * i;
      if (part < chunks_per_key) *reinterpret_cast<uint4*>(kt + my_key * ldk + 8 * part) = pre[i];
    }
    __syncthreads();
    // the values' copy, transposed: a thread takes two neighbouring keys and eight columns, and
    // writes eight pairs. Within a transposed row the keys stand in the order in which the second
    // product sums them: key 16 hi + 4 g + lo at place 8 g + 4 hi + lo, so that a lane's eight are
    // 16 bytes in a row. Lanes side by side take key pairs side by side.
    for (int item = threadIdx.x; item < (LMA_BN / 2) * (Dv >> 3); item += 256 * HALVES) {
      const int j = (item & 15) * 2, d0 = (item >> 4) * 8;
      LatPack v0, v1;
      v0.u = *reinterpret_cast<const uint4*>(kt + j * ldk + d0);
      v1.u = *reinterpret_cast<const uint4*>(kt + (j + 1) * ldk + d0);
      const int place = 8 * ((j >> 2) & 3) + 4 * (j >> 4) + (j & 3);
      unsigned* dst = reinterpret_cast<unsigned*>(reinterpret_cast<unsigned short*>(vt) + d0 * LMA_VLD + place);
      const unsigned short* e0 = reinterpret_cast<const unsigned short*>(&v0.u);
      const unsigned short* e1 = reinterpret_cast<const unsigned short*>(&v1.u);
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i * (LMA_VLD / 2)] = (unsigned)e0[i] | ((unsigned)e1[i] << 16);
    }
    if (kt0 + LMA_BN < k_end) {                               // the next tile travels while this one is worked on
      fetch(kt0 + LMA_BN, next_page);
      next_page = lookup(kt0 + 2 * LMA_BN);
    }
    __syncthreads();
    if (!wave_active || kt0 >= wave_k_end || kt0 + LMA_BN <= wave_k_begin) continue;
    // the two halves of the tile are two chains of matrix instructions that take turns, and the
    // operands of three steps are asked for together, so that neither a read nor a result is waited for alone
    lat_f32x4_t sc[2] = {lat_f32x4_t{0.f, 0.f, 0.f, 0.f}, lat_f32x4_t{0.f, 0.f, 0.f, 0.f}};
    {
      const bf16_t* kr0 = kt + col * ldk + 8 * grp;
      const bf16_t* kr1 = kr0 + 16 * ldk;
#pragma unroll
      for (int i0 = 0; i0 < KS; i0 += 3) {
        LatPack a0[3], a1[3];
#pragma unroll
        for (int u = 0; u < 3; ++u) {
          if (i0 + u < KS && i0 + u < ks) {
            a0[u].u = *reinterpret_cast<const uint4*>(kr0 + 32 * (i0 + u));
            a1[u].u = *reinterpret_cast<const uint4*>(kr1 + 32 * (i0 + u));
          }
        }
#pragma unroll
        for (int u = 0; u < 3; ++u) {
          if (i0 + u < KS && i0 + u < ks) {
            sc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[u].v, qreg[i0 + u].v, sc[0], 0, 0, 0);
            sc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[u].v, qreg[i0 + u].v, sc[1], 0, 0, 0);
          }
        }
      }
    }
    float v[8];
    // a tile that every row of the wavefront sees whole needs no masks
    const bool whole = wave_full && kt0 + LMA_BN <= k_end && kt0 + LMA_BN - 1 <= wave_first_pos &&
                       (window <= 0 || wave_last_pos - kt0 < window);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = sc[j >> 2][j & 3];
    if (!whole) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = kt0 + 16 * (j >> 2) + 4 * grp + (j & 3);
        bool seen = valid && key <= pos && key < k_end;
        if (window > 0 && pos - key >= window) seen = false;
        if (!seen) v[j] = -INFINITY;
      }
    }
    float mx = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
    mx = quad_rows_max(mx);
    // The exponent's reference m_run follows the row's maximum only when that has grown by more
    // than 8 (a factor of 256) since it was set: weights then stay below 256, which float32 sums and
    // bfloat16 weights carry as well as numbers below 1, and the sums are rescaled a few times a row
    // instead of once a tile. The result is the same quotient.
    const float m_tile = mx * scale_log2;
    const bool rescale = m_tile > m_run + 8.f;                // also the first tile in which the row sees a key
    float alpha = 1.f;
    if (rescale) {
      alpha = __builtin_amdgcn_exp2f(m_run - m_tile);         // 0 from minus infinity
      m_run = m_tile;
    }
    LatPack p;
    float sum = 0.f;
    if (m_run > -INFINITY) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float e = __builtin_amdgcn_exp2f(fmaf(v[j], scale_log2, -m_run));   // 2^x; results below the normal range are zero
        sum += e;
        p.e[j] = (__bf16)e;
      }
    } else {
      p.u = make_uint4(0, 0, 0, 0);
    }
    sum = quad_rows_sum(sum);
    l_run = l_run * alpha + sum;
    const bool moved = __builtin_amdgcn_ballot_w64(rescale) != 0;
#pragma unroll
    for (int nb = 0; nb < NV; ++nb) {
      if (nb < nv) {
        if (moved) acc[nb] *= alpha;
        LatPack a;
        a.u = *reinterpret_cast<const uint4*>(vt + (16 * (nb0 + nb) + col) * LMA_VLD + 8 * grp);
        acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, p.v, acc[nb], 0, 0, 0);
      }
    }
  }
  if (!valid) return;
  if (splits > 1) {
    float* dst = partial + (((size_t)(q0 + tok) * H + head) * splits + blockIdx.y) * (Dv + 2);
    if (grp == 0 && half == 0) {
      dst[Dv] = m_run;
      dst[Dv + 1] = l_run;
    }
#pragma unroll
    for (int nb = 0; nb < NV; ++nb) {
      if (nb < nv) *reinterpret_cast<float4*>(dst + 16 * (nb0 + nb) + 4 * grp) = make_float4(acc[nb][0], acc[nb][1], acc[nb][2], acc[nb][3]);
    }
    return;
  }
  // the sink joins where the row's sum is final: exp(sink) against the exponent's reference
  if (sink) l_run += __builtin_amdgcn_exp2f(fmaf(sink[head], 1.44269504088896341f, -m_run));
  float inv = 1.f / l_run;
  if (gate) inv /= 1.f + expf(-bf16_to_float(gate[(size_t)(q0 + tok) * gate_stride + head]));
  bf16_t* o = out + ((size_t)(q0 + tok) * H + head) * Dv + 4 * grp;
#pragma unroll
  for (int nb = 0; nb < NV; ++nb) {
    if (nb < nv) {
      union {
        uint2 u;
        bf16_t e[4];
      } pk;
#pragma unroll
      for (int i = 0; i < 4; ++i) pk.e[i] = float_to_bf16(acc[nb][i] * inv);
      *reinterpret_cast<uint2*>(o + 16 * (nb0 + nb)) = pk.u;
    }
  }
}

// out[row] = sum_s 2^(m_s - m) acc_s / sum_s 2^(m_s - m) l_s, m = max_s m_s, the shares in their order;
// the sink's term joins the denominator and the gate multiplies the quotient, as in the kernels above.
__global__ void latent_attn_merge_kernel(const float* __restrict__ partial, bf16_t* __restrict__ out, int Dv, int splits,
                                         int H, const float* __restrict__ sink, const bf16_t* __restrict__ gate,
                                         long gate_stride) {
  const size_t row = blockIdx.x;
  const float* src = partial + row * splits * (Dv + 2);
  float m = -INFINITY;
  for (int s = 0; s < splits; ++s) m = fmaxf(m, src[(size_t)s * (Dv + 2) + Dv]);
  float l = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float ms = src[(size_t)s * (Dv + 2) + Dv];
    if (ms > -INFINITY) l += exp2f(ms - m) * src[(size_t)s * (Dv + 2) + Dv + 1];
  }
  if (sink) l += exp2f(sink[row % H] * 1.44269504088896341f - m);
  float inv = 1.f / l;
  if (gate) inv /= 1.f + expf(-bf16_to_float(gate[(row / H) * gate_stride + row % H]));
  for (int d = threadIdx.x; d < Dv; d += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float ms = src[(size_t)s * (Dv + 2) + Dv];
      if (ms > -INFINITY) a += exp2f(ms - m) * src[(size_t)s * (Dv + 2) + d];
    }
    out[row * Dv + d] = float_to_bf16(a * inv);
  }
}

static int raise_shared_memory(const void* kernel, size_t smem) {
  if (smem <= 48 * 1024) return 0;
  if (smem > 160 * 1024) return Q3_ERR_UNSUPPORTED;
  return (int)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
}

extern "C" int q3_latent_prepare(const void* down, long down_stride, int T, int q_rank, int kv_rank, int rot_dim, const void* q_weight,
                                 const void* kv_weight, int w_dtype, float eps, const float* inv_freq, int rot_pairs,
                                 float rot_factor, const int* positions, const int* seq_index,
                                 const int* block_table, int bt_stride, int bt_rows, void* cache, int page,
                                 int num_pages, void* cq, int dtype, hipStream_t stream) {
  if (T <= 0 || q_rank <= 0 || kv_rank <= 0 || rot_dim < 0 || 2 * rot_pairs > rot_dim || rot_pairs < 0)
    return Q3_ERR_BAD_ARGUMENT;
  if (down_stride < q_rank + kv_rank + rot_dim || (rot_pairs > 0 && !inv_freq)) return Q3_ERR_BAD_ARGUMENT;
  if (cache && (!block_table || page <= 0 || num_pages <= 0 || bt_stride <= 0)) return Q3_ERR_BAD_ARGUMENT;
  const int R = q_rank + kv_rank + rot_dim;
  const size_t smem = (size_t)(32 + R) * sizeof(float);
  int threads = 64;
  while (threads < 512 && threads * 2 < R) threads *= 2;
  Q3_DISPATCH_DTYPE(dtype, TT, Q3_DISPATCH_DTYPE(w_dtype, WW, {
    int e = raise_shared_memory((const void*)latent_prepare_kernel<TT, WW>, smem);
    if (e) return e;
    hipLaunchKernelGGL((latent_prepare_kernel<TT, WW>), dim3(T), dim3(threads), smem, stream, (const TT*)down, down_stride,
                       q_rank, kv_rank, rot_dim, (const WW*)q_weight, (const WW*)kv_weight, eps, inv_freq, rot_pairs,
                       rot_factor, positions, seq_index, block_table, bt_stride, bt_rows, (TT*)cache, page, num_pages,
                       (TT*)cq);
    return q3_launch_status();
  }));
  return Q3_ERR_BAD_ARGUMENT;
}

extern "C" int q3_headwise_linear(const void* x, long x_row, int x_head, const void* w, void* out, long out_row,
                                  int out_head, int n_rows, int H, int I, int O, int dtype, int matrix_cores,
                                  hipStream_t stream) {
  if (n_rows <= 0 || H <= 0 || I <= 0 || O <= 0 || H > 65535) return Q3_ERR_BAD_ARGUMENT;
  if (matrix_cores) {
    // the caller has checked: bfloat16, I in steps of 32, rows of x at multiples of 16 bytes
    if (dtype != Q3_BF16 || I % 32 || x_row % 8 || x_head % 8 || ((uintptr_t)x & 15) || ((uintptr_t)w & 15))
      return Q3_ERR_BAD_ARGUMENT;
    const int zs = (O + 127) / 128;
    if (n_rows > 64) {
      hipLaunchKernelGGL(headwise_linear_mma_kernel<2>, dim3((n_rows + 127) / 128, H, zs), dim3(256), 0, stream,
                         (const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)out, out_row, out_head, n_rows, I, O);
    } else {
      hipLaunchKernelGGL(headwise_linear_mma_kernel<1>, dim3((n_rows + 63) / 64, H, zs), dim3(256), 0, stream,
                         (const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)out, out_row, out_head, n_rows, I, O);
    }
    return q3_launch_status();
  }
  const size_t smem = (size_t)16 * I * sizeof(float);
  int threads = 64;
  while (threads < 256 && threads < O) threads *= 2;
  const dim3 grid((n_rows + 15) / 16, H, (O + threads - 1) / threads);
  Q3_DISPATCH_DTYPE(dtype, TT, {
    int e = raise_shared_memory((const void*)headwise_linear_kernel<TT>, smem);
    if (e) return e;
    hipLaunchKernelGGL(headwise_linear_kernel<TT>, grid, dim3(threads), smem, stream, (const TT*)x, x_row, x_head,
                       (const TT*)w, (TT*)out, out_row, out_head, n_rows, I, O);
  });
  return q3_launch_status();
}

extern "C" int q3_rotate_heads(const void* x, long x_row, int x_head, void* out, long out_row, int out_head, int T,
                               int H, int rot_dim, int rot_pairs, const float* inv_freq, float rot_factor,
                               const int* positions, int dtype, hipStream_t stream) {
  if (T <= 0 || H <= 0 || rot_dim <= 0 || rot_pairs < 0 || 2 * rot_pairs > rot_dim) return Q3_ERR_BAD_ARGUMENT;
  const int work = H * ((rot_dim + 1) / 2);
  int threads = 64;
  while (threads < 256 && threads < work) threads *= 2;
  Q3_DISPATCH_DTYPE(dtype, TT,
                    hipLaunchKernelGGL(rotate_heads_kernel<TT>, dim3(T), dim3(threads), 0, stream, (const TT*)x, x_row,
                                       x_head, (TT*)out, out_row, out_head, H, rot_dim, rot_pairs, inv_freq,
                                       rot_factor, positions));
  return q3_launch_status();
}

template <typename T, int NV>
static int launch_latent_attn(const void* q, void* out, const void* cache, int num_pages, const int* block_table,
                              int bt_stride, const int* cu_q, const int* kv_lens, int B, int H, int Dk, int Dv,
                              int page, float scale, int window, int max_q_len, const float* sink, const void* gate,
                              long gate_stride, hipStream_t stream) {
  const size_t smem = (size_t)(LAT_BM * Dk + LAT_BN * (Dk + 1) + LAT_BM * (LAT_BN + 1)) * sizeof(float);
  int e = raise_shared_memory((const void*)latent_attn_kernel<T, NV>, smem);
  if (e) return e;
  const long tiles = ((long)max_q_len * H + LAT_BM - 1) / LAT_BM;
  if (tiles > 0x7fffffffL || B > 65535) return Q3_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((latent_attn_kernel<T, NV>), dim3((unsigned)tiles, B), dim3(256), smem, stream, (const T*)q,
                     (T*)out, (const T*)cache, num_pages, block_table, bt_stride, cu_q, kv_lens, H, Dk, Dv, page, scale,
                     window, sink, (const T*)gate, gate_stride);
  return q3_launch_status();
}

template <int KS, int NV, int HALVES>
static int launch_latent_attn_mma(const void* q, void* out, const void* cache, int num_pages, const int* block_table,
                                  int bt_stride, const int* cu_q, const int* kv_lens, int B, int T, int H, int Dk,
                                  int Dv, int page, float scale, int window, int splits, float* partial,
                                  const float* sink, const void* gate, long gate_stride, hipStream_t stream) {
  const size_t smem = (size_t)(LMA_BN * (Dk + LMA_KPAD) + Dv * LMA_VLD) * sizeof(bf16_t);
  int e = raise_shared_memory((const void*)latent_attn_mma_kernel<KS, NV, HALVES>, smem);
  if (e) return e;
  const long tiles = ((long)T * H) / LMA_ROWS + B;            // at least the sequences' tiles of 64 rows together
  if (tiles > 0x7fffffffL || splits < 1 || splits > 65535 || (splits > 1 && !partial)) return Q3_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((latent_attn_mma_kernel<KS, NV, HALVES>), dim3((unsigned)tiles, splits), dim3(256 * HALVES), smem, stream,
                     (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, num_pages, block_table, bt_stride, cu_q,
                     kv_lens, B, H, Dk, Dv, page, scale * 1.44269504088896341f, window, splits, partial, sink,
                     (const bf16_t*)gate, gate_stride);
  if (splits > 1)
    hipLaunchKernelGGL(latent_attn_merge_kernel, dim3((unsigned)((long)T * H)), dim3(Dv >= 256 ? 256 : 64), 0, stream,
                       partial, (bf16_t*)out, Dv, splits, H, sink, (const bf16_t*)gate, gate_stride);
  return q3_launch_status();
}

// Whether the matrix-core kernel serves these sizes.
extern "C" int q3_latent_attention_fast_path(int Dk, int Dv, int dtype) {
  return dtype == Q3_BF16 && Dk % 32 == 0 && Dv % 16 == 0 && Dv <= Dk && Dk <= 576 && Dv <= 512;
}

extern "C" int q3_latent_attention(const void* q, void* out, const void* cache, int num_pages, const int* block_table,
                                   int bt_stride, const int* cu_q, const int* kv_lens, int B, int T, int H, int Dk,
                                   int Dv, int page, float scale, int window, int max_q_len, int dtype, int general,
                                   int splits, float* partial, const float* sink, const void* gate, long gate_stride,
                                   hipStream_t stream) {
  if (B <= 0 || T <= 0 || H <= 0 || Dk <= 0 || Dv <= 0 || Dv > Dk || page <= 0 || max_q_len <= 0 || window < 0)
    return Q3_ERR_BAD_ARGUMENT;
  if (Dv > 1024) return Q3_ERR_UNSUPPORTED;
  if (gate && gate_stride < H) return Q3_ERR_BAD_ARGUMENT;
  if (!general && q3_latent_attention_fast_path(Dk, Dv, dtype)) {
    if (Dk <= 192 && Dv <= 128)
      return launch_latent_attn_mma<6, 8, 1>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, T, H, Dk,
                                          Dv, page, scale, window, splits, partial, sink, gate, gate_stride, stream);
    if (Dk <= 320 && Dv <= 256)
      return launch_latent_attn_mma<10, 16, 1>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, T, H,
                                            Dk, Dv, page, scale, window, splits, partial, sink, gate, gate_stride, stream);
    return launch_latent_attn_mma<18, 16, 2>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, T, H, Dk,
                                          Dv, page, scale, window, splits, partial, sink, gate, gate_stride, stream);
  }
  Q3_DISPATCH_DTYPE(dtype, TT, {
    if (Dv <= 128)
      return launch_latent_attn<TT, 8>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, H, Dk, Dv,
                                       page, scale, window, max_q_len, sink, gate, gate_stride, stream);
    if (Dv <= 256)
      return launch_latent_attn<TT, 16>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, H, Dk, Dv,
                                        page, scale, window, max_q_len, sink, gate, gate_stride, stream);
    if (Dv <= 512)
      return launch_latent_attn<TT, 32>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, H, Dk, Dv,
                                        page, scale, window, max_q_len, sink, gate, gate_stride, stream);
    return launch_latent_attn<TT, 64>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, H, Dk, Dv,
                                      page, scale, window, max_q_len, sink, gate, gate_stride, stream);
  });
  return Q3_ERR_BAD_ARGUMENT;
}
