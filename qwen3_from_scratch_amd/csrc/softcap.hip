// Softmax attention with biased projections, a norm over the whole query and key projections,
// a rotation of neighbouring pairs, capped scores, key and value heads of different sizes and a
// gate per head, over a paged cache: keys (pages, G, page, dim), values (pages, G, page, vdim) or,
// transposed within the page as the matrix-core kernels read them, (pages, G, vdim, page).
#include "common.h"

// One block per token. The row is [q: H dim | k: G dim | v: G vdim | ...] float32, `bias` covers
// q, k and v (null: projections without biases). q and k (bias added) are each divided by the root mean square of the whole
// projection and multiplied by their weight, then the first 2 * half numbers of every head turn
// in pairs (2i, 2i + 1) by position * inv_freq[i]. q goes to `q_out`, k and v (bias added) into
// the token's place in the cache, when one is given.
template <typename TA>
__global__ void softcap_prepare_kernel(const float* __restrict__ rows, long row_stride, const float* __restrict__ bias,
                                       const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
                                       const float* __restrict__ inv_freq, int half, const int* __restrict__ positions,
                                       const int* __restrict__ seq_index, const int* __restrict__ block_table,
                                       int table_width, TA* __restrict__ k_cache, TA* __restrict__ v_cache, int page,
                                       TA* __restrict__ q_out, int H, int G, int dim, int vdim, int v_transposed) {
  __shared__ float scratch[17];
  const int t = blockIdx.x;
  const float* row = rows + (size_t)t * row_stride;
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  float sq = 0.f, sk = 0.f;
  for (int j = threadIdx.x; j < nq; j += blockDim.x) {
    const float z = row[j] + (bias ? bias[j] : 0.f);
    sq += z * z;
  }
  for (int j = threadIdx.x; j < nk; j += blockDim.x) {
    const float z = row[nq + j] + (bias ? bias[nq + j] : 0.f);
    sk += z * z;
  }
  const float rq = rsqrtf(block_sum(sq, scratch) / (float)nq + eps);
  const float rk = rsqrtf(block_sum(sk, scratch) / (float)nk + eps);
  const int pos = positions[t];
  const float fpos = (float)pos;
  for (int j = threadIdx.x; j < nq; j += blockDim.x) {
    const int e = j % dim;
    float own = (row[j] + (bias ? bias[j] : 0.f)) * rq * q_weight[j];
    if (e < 2 * half) {
      const int p = j ^ 1;
      const float other = (row[p] + (bias ? bias[p] : 0.f)) * rq * q_weight[p];
      const float angle = fpos * inv_freq[e >> 1];
      const float c = cosf(angle), s = sinf(angle);
      own = (e & 1) ? own * c + other * s : own * c - other * s;
    }
    q_out[(size_t)t * nq + j] = from_float<TA>(own);
  }
  if (!k_cache) return;
  const int pg = block_table[(size_t)seq_index[t] * table_width + pos / page];
  if (pg < 0) return;
  const int off = pos % page;
  for (int j = threadIdx.x; j < nk; j += blockDim.x) {
    const int g = j / dim, e = j % dim;
    float own = (row[nq + j] + (bias ? bias[nq + j] : 0.f)) * rk * k_weight[j];
    if (e < 2 * half) {
      const int p = j ^ 1;
      const float other = (row[nq + p] + (bias ? bias[nq + p] : 0.f)) * rk * k_weight[p];
      const float angle = fpos * inv_freq[e >> 1];
      const float c = cosf(angle), s = sinf(angle);
      own = (e & 1) ? own * c + other * s : own * c - other * s;
    }
    k_cache[(((size_t)pg * G + g) * page + off) * dim + e] = from_float<TA>(own);
  }
  for (int j = threadIdx.x; j < nv; j += blockDim.x) {
    const int g = j / vdim, e = j % vdim;
    const size_t at = v_transposed ? (((size_t)pg * G + g) * vdim + e) * page + off
                                   : (((size_t)pg * G + g) * page + off) * vdim + e;
    v_cache[at] = from_float<TA>(row[nq + nk + j] + (bias ? bias[nq + nk + j] : 0.f));
  }
}

// The general form: one wavefront per (token, head). Keys are taken in tiles of 64 that start at
// absolute positions in steps of 64, one key a lane: score = (q . k) scale, capped as
// cap * tanh(score / cap) when cap > 0; running maximum and sum in float32; then every lane sums
// its columns of the values with the tile's weights. The result is divided by the sum and
// multiplied by sigmoid(gate[t, h]) when a gate is given. With `sink` (H floats) the sum also holds
// exp(sink[h]), a term that has no key and no value and is not scaled.
#define Q3_CAP_DIM_MOST 512
#define Q3_CAP_VSLICES 8
template <typename TA>
__global__ void __launch_bounds__(64) softcap_attention_kernel(
    const TA* __restrict__ q, const TA* __restrict__ k_cache, const TA* __restrict__ v_cache,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ seq_index,
    const int* __restrict__ positions, float scale, float cap, int window, const float* __restrict__ gate,
    long gate_stride, TA* __restrict__ out, int H, int G, int dim, int vdim, int page, int v_transposed,
    const float* __restrict__ sink) {
  __shared__ float sq[Q3_CAP_DIM_MOST];
  __shared__ float sp[64];
  const int lane = threadIdx.x;
  const int t = blockIdx.x, h = blockIdx.y;
  const int g = h / (H / G);
  const int pos = positions[t];
  const int* table = block_table + (size_t)seq_index[t] * table_width;
  const TA* qr = q + ((size_t)t * H + h) * dim;
  for (int e = lane; e < dim; e += 64) sq[e] = to_float(qr[e]);
  __syncthreads();
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[Q3_CAP_VSLICES];
#pragma unroll
  for (int i = 0; i < Q3_CAP_VSLICES; ++i) acc[i] = 0.f;
  for (int j0 = lo / 64 * 64; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j >= lo && j <= pos;
    float s = -INFINITY;
    if (valid) {
      const int pg = table[j / page];
      const TA* kr = k_cache + (((size_t)(pg < 0 ? 0 : pg) * G + g) * page + j % page) * dim;
      float dot = 0.f;
      for (int e = 0; e < dim; ++e) dot += sq[e] * to_float(kr[e]);
      s = dot * scale;
      if (cap > 0.f) s = cap * tanhf(s / cap);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float keep = m == -INFINITY ? 0.f : expf(m - m_new);
    l = l * keep + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < Q3_CAP_VSLICES; ++i) acc[i] *= keep;
    sp[lane] = p;
    __syncthreads();
    const int last = pos - j0 < 63 ? pos - j0 : 63;
    for (int jj = (lo > j0 ? lo - j0 : 0); jj <= last; ++jj) {
      const float pj = sp[jj];
      const int key = j0 + jj;
      const int pg = table[key / page];
      const size_t head = (size_t)(pg < 0 ? 0 : pg) * G + g;
      const TA* vr = v_transposed ? v_cache + head * vdim * page + key % page : v_cache + (head * page + key % page) * vdim;
      const int apart = v_transposed ? page : 1;
#pragma unroll
      for (int i = 0; i < Q3_CAP_VSLICES; ++i) {
        const int c = lane + 64 * i;
        if (c < vdim) acc[i] += pj * to_float(vr[(size_t)c * apart]);
      }
    }
    __syncthreads();
  }
  const float open = gate ? 1.f / (1.f + expf(-gate[(size_t)t * gate_stride + h])) : 1.f;
  if (sink) l += expf(sink[h] - m);
  const float norm = open / l;
#pragma unroll
  for (int i = 0; i < Q3_CAP_VSLICES; ++i) {
    const int c = lane + 64 * i;
    if (c < vdim) out[((size_t)t * H + h) * vdim + c] = from_float<TA>(acc[i] * norm);
  }
}

// Queries, keys and values with a norm per head: one block per token, a wavefront per head in turn.
// The row is [q: H dim | k: G dim | v: G vdim | ...] float32, or [q: H dim | ...] for a layer that
// makes no keys of its own (`G` 0). Every head of q (of k) is divided by its own root mean square
// and multiplied by `q_weight` (`k_weight`), dim numbers that all heads share; no rotation. q goes
// to `q_out`, k and v into the token's place in the cache.
template <typename TA>
__global__ void __launch_bounds__(256) headnorm_prepare_kernel(
    const float* __restrict__ rows, long row_stride, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, float eps, const int* __restrict__ positions, const int* __restrict__ seq_index,
    const int* __restrict__ block_table, int table_width, TA* __restrict__ k_cache, TA* __restrict__ v_cache, int page,
    TA* __restrict__ q_out, int H, int G, int dim, int vdim, int v_transposed) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / Q3_WAVE, lane = threadIdx.x % Q3_WAVE, waves = blockDim.x / Q3_WAVE;
  const float* row = rows + (size_t)t * row_stride;
  const int nq = H * dim, nk = G * dim;
  for (int h = wave; h < H; h += waves) {
    const float* src = row + (size_t)h * dim;
    float acc = 0.f;
    for (int e = lane; e < dim; e += Q3_WAVE) acc += src[e] * src[e];
    const float r = rsqrtf(wave_sum(acc) / (float)dim + eps);
    for (int e = lane; e < dim; e += Q3_WAVE) q_out[(size_t)t * nq + h * dim + e] = from_float<TA>(src[e] * r * q_weight[e]);
  }
  if (G == 0) return;
  const int pos = positions[t];
  const int pg = block_table[(size_t)seq_index[t] * table_width + pos / page];
  if (pg < 0) return;
  const int off = pos % page;
  for (int g = wave; g < G; g += waves) {
    const float* src = row + nq + (size_t)g * dim;
    float acc = 0.f;
    for (int e = lane; e < dim; e += Q3_WAVE) acc += src[e] * src[e];
    const float r = rsqrtf(wave_sum(acc) / (float)dim + eps);
    for (int e = lane; e < dim; e += Q3_WAVE)
      k_cache[(((size_t)pg * G + g) * page + off) * dim + e] = from_float<TA>(src[e] * r * k_weight[e]);
    const float* val = row + nq + nk + (size_t)g * vdim;
    for (int e = lane; e < vdim; e += Q3_WAVE) {
      const size_t at = v_transposed ? (((size_t)pg * G + g) * vdim + e) * page + off
                                     : (((size_t)pg * G + g) * page + off) * vdim + e;
      v_cache[at] = from_float<TA>(val[e]);
    }
  }
}

extern "C" int q3_headnorm_prepare(const float* rows, long row_stride, const float* q_weight, const float* k_weight,
                                   float eps, const int* positions, const int* seq_index, const int* block_table,
                                   int table_width, void* k_cache, void* v_cache, int page, void* q_out, int T, int H,
                                   int G, int dim, int vdim, int v_transposed, int act_dtype, hipStream_t stream) {
  if (T <= 0 || H <= 0 || G < 0 || dim <= 0 || vdim <= 0 || !q_weight) return Q3_ERR_BAD_ARGUMENT;
  if (G > 0 && (H % G || !k_weight || !k_cache || !v_cache || !block_table || page <= 0 || table_width <= 0))
    return Q3_ERR_BAD_ARGUMENT;
  Q3_DISPATCH_DTYPE(act_dtype, TA,
                    hipLaunchKernelGGL(headnorm_prepare_kernel<TA>, dim3(T), dim3(256), 0, stream, rows, row_stride,
                                       q_weight, k_weight, eps, positions, seq_index, block_table, table_width,
                                       (TA*)k_cache, (TA*)v_cache, page, (TA*)q_out, H, G, dim, vdim, v_transposed));
  return q3_launch_status();
}

// out[t, h, :] *= sigmoid(gate[t, h]) for a result that another kernel has left ungated.
template <typename TA>
__global__ void gate_heads_kernel(TA* __restrict__ out, const float* __restrict__ gate, long gate_stride, int H, int vdim) {
  const int t = blockIdx.x;
  for (int e = threadIdx.x; e < H * vdim; e += blockDim.x) {
    const float open = 1.f / (1.f + expf(-gate[(size_t)t * gate_stride + e / vdim]));
    out[(size_t)t * H * vdim + e] = from_float<TA>(to_float(out[(size_t)t * H * vdim + e]) * open);
  }
}

extern "C" int q3_gate_heads(void* out, const float* gate, long gate_stride, int T, int H, int vdim, int act_dtype,
                             hipStream_t stream) {
  if (T <= 0 || H <= 0 || vdim <= 0) return Q3_ERR_BAD_ARGUMENT;
  Q3_DISPATCH_DTYPE(act_dtype, TA, hipLaunchKernelGGL(gate_heads_kernel<TA>, dim3(T), dim3(256), 0, stream, (TA*)out,
                                                      gate, gate_stride, H, vdim));
  return q3_launch_status();
}

extern "C" int q3_softcap_prepare(const float* rows, long row_stride, const float* bias, const float* q_weight,
                                  const float* k_weight, float eps, const float* inv_freq, int half,
                                  const int* positions, const int* seq_index, const int* block_table, int table_width,
                                  void* k_cache, void* v_cache, int page, void* q_out, int T, int H, int G, int dim,
                                  int vdim, int v_transposed, int act_dtype, hipStream_t stream) {
  if (T <= 0 || H <= 0 || G <= 0 || H % G || dim <= 0 || vdim <= 0 || half < 0 || 2 * half > dim) return Q3_ERR_BAD_ARGUMENT;
  if (half > 0 && !inv_freq) return Q3_ERR_BAD_ARGUMENT;
  if (k_cache && (!v_cache || !block_table || page <= 0 || table_width <= 0)) return Q3_ERR_BAD_ARGUMENT;
  Q3_DISPATCH_DTYPE(act_dtype, TA,
                    hipLaunchKernelGGL(softcap_prepare_kernel<TA>, dim3(T), dim3(256), 0, stream, rows, row_stride, bias,
                                       q_weight, k_weight, eps, inv_freq, half, positions, seq_index, block_table,
                                       table_width, (TA*)k_cache, (TA*)v_cache, page, (TA*)q_out, H, G, dim, vdim,
                                       v_transposed));
  return q3_launch_status();
}

extern "C" int q3_softcap_attention(const void* q, const void* k_cache, const void* v_cache, const int* block_table,
                                    int table_width, const int* seq_index, const int* positions, float scale, float cap,
                                    int window, const float* gate, long gate_stride, void* out, int T, int H, int G,
                                    int dim, int vdim, int page, int v_transposed, const float* sink, int act_dtype,
                                    hipStream_t stream) {
  if (T <= 0 || H <= 0 || G <= 0 || H % G || dim <= 0 || vdim <= 0 || page <= 0 || table_width <= 0 || window < 0 ||
      H > 65535)
    return Q3_ERR_BAD_ARGUMENT;
  if (dim > Q3_CAP_DIM_MOST || vdim > 64 * Q3_CAP_VSLICES) return Q3_ERR_UNSUPPORTED;
  Q3_DISPATCH_DTYPE(act_dtype, TA,
                    hipLaunchKernelGGL(softcap_attention_kernel<TA>, dim3(T, H), dim3(64), 0, stream, (const TA*)q,
                                       (const TA*)k_cache, (const TA*)v_cache, block_table, table_width, seq_index,
                                       positions, scale, cap, window, gate, gate_stride, (TA*)out, H, G, dim, vdim,
                                       page, v_transposed, sink));
  return q3_launch_status();
}
