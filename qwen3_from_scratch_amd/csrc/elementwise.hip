// Embedding row gather and the gated activations (SwiGLU and its gelu forms).
#include "common.h"

// out[t, :] = float(table[ids[t], :]) * scale. An id outside the table gives a row of
// zeros (the host refuses such ids before launching; this only keeps the
// kernel inside its operands).
template <typename T>
__global__ void embed_rows_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                  float* __restrict__ out, int H, int V, float scale) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;
  const T* row = table + (size_t)(ok ? id : 0) * H;
  float* dst = out + (size_t)t * H;
  for (int j = threadIdx.x; j < H; j += blockDim.x) dst[j] = ok ? to_float(row[j]) * scale : 0.f;
}

// out[t, j] = act(gate[t, j]) * up[t, j] for rows that interleave the two:
// gate_up[t, 2j] = gate[t, j], gate_up[t, 2j + 1] = up[t, j]. ACT 0: silu(g) = g / (1 + exp(-g));
// 1: the tanh form of gelu, 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))); 2: the exact gelu,
// 0.5 g (1 + erf(g / sqrt 2)). Evaluated in float32 and rounded once.
template <int ACT>
__device__ inline float gate_value(float g) {
  if (ACT == 0) return g / (1.f + expf(-g));
  if (ACT == 1) return 0.5f * g * (1.f + tanhf(0.79788456080286536f * (g + 0.044715f * g * g * g)));
  return 0.5f * g * (1.f + erff(g * 0.70710678118654752f));
}

template <typename T, int ACT>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= I) return;
  const T* row = gate_up + (size_t)t * 2 * I;
  const float g = to_float(row[2 * j]);
  const float u = to_float(row[2 * j + 1]);
  out[(size_t)t * I + j] = from_float<T>(gate_value<ACT>(g) * u);
}

// The same, eight outputs per thread with 16-byte loads and stores; bfloat16, I a multiple of 8.
template <int ACT>
__global__ void swiglu_vec8_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const int j = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (j >= I) return;
  const bf16_t* row = gate_up + (size_t)t * 2 * I + 2 * j;
  union {
    uint4 u;
    bf16_t e[8];
  } a, b, o;
  a.u = *reinterpret_cast<const uint4*>(row);
  b.u = *reinterpret_cast<const uint4*>(row + 8);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = bf16_to_float(a.e[2 * i]), g1 = bf16_to_float(b.e[2 * i]);
    o.e[i] = float_to_bf16(gate_value<ACT>(g0) * bf16_to_float(a.e[2 * i + 1]));
    o.e[4 + i] = float_to_bf16(gate_value<ACT>(g1) * bf16_to_float(b.e[2 * i + 1]));
  }
  *reinterpret_cast<uint4*>(out + (size_t)t * I + j) = o.u;
}

// A gated unit with clamped branches over rows that interleave the two (in[t, 2j] the gate's, in[t, 2j + 1]
// the other branch's): a = in * w + bias with w = scale[scale_index[t]] (or scale[t]; 1 without a scale) and
// a float32 bias over the interleaved columns (or none); g = min(a_gate, limit), u = clamp(a_up, -limit, limit);
// out[t, j] = g * sigmoid(slope * g) * (u + 1). float32 throughout, rounded once; the input may be
// float32 where the output is not (a product that left its sums unrounded).
template <typename T, typename TO>
__global__ void glu_clamped_kernel(const T* __restrict__ in, const float* __restrict__ bias,
                                   const float* __restrict__ scale, const int* __restrict__ scale_index,
                                   TO* __restrict__ out, int T_rows, int I, float limit, float slope) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= I) return;
  const float bg = bias ? bias[2 * j] : 0.f, bu = bias ? bias[2 * j + 1] : 0.f;
  for (int t = blockIdx.y; t < T_rows; t += gridDim.y) {
    const float w = scale ? scale[scale_index ? scale_index[t] : t] : 1.f;
    const T* row = in + (size_t)t * 2 * I;
    float g = to_float(row[2 * j]) * w + bg;
    float u = to_float(row[2 * j + 1]) * w + bu;
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    out[(size_t)t * I + j] = from_float<TO>(g / (1.f + expf(-slope * g)) * (u + 1.f));
  }
}

extern "C" int q3_glu_clamped(const void* in, const float* bias, const float* scale, const int* scale_index, void* out,
                              int T, int I, float limit, float slope, int dtype, int out_dtype, hipStream_t stream) {
  if (T <= 0 || I <= 0 || !(limit > 0.f) || (scale_index && !scale)) return Q3_ERR_BAD_ARGUMENT;
  const int threads = I >= 256 ? 256 : 64;
  const dim3 grid((I + threads - 1) / threads, T < 65535 ? T : 65535);
  Q3_DISPATCH_DTYPE(dtype, TT, Q3_DISPATCH_DTYPE(out_dtype, TO, {
                      hipLaunchKernelGGL((glu_clamped_kernel<TT, TO>), grid, dim3(threads), 0, stream, (const TT*)in, bias,
                                         scale, scale_index, (TO*)out, T, I, limit, slope);
                    }));
  return q3_launch_status();
}

extern "C" int q3_embed_rows(const int* ids, const void* table, float* out, int T, int H, int V, float scale,
                             int table_dtype, hipStream_t stream) {
  if (T <= 0 || H <= 0 || V <= 0) return Q3_ERR_BAD_ARGUMENT;
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  Q3_DISPATCH_DTYPE(table_dtype, TT,
                    hipLaunchKernelGGL(embed_rows_kernel<TT>, dim3(T), dim3(threads), 0, stream, ids,
                                       (const TT*)table, out, H, V, scale));
  return q3_launch_status();
}

template <int ACT>
static int launch_gated_act(const void* gate_up, void* out, int T, int I, int dtype, hipStream_t stream) {
  const int threads = 256;
  // blockIdx.y carries the row; rows beyond 65535 are covered by several launches
  for (int t0 = 0; t0 < T; t0 += 65535) {
    const int rows = T - t0 < 65535 ? T - t0 : 65535;
    if (dtype == Q3_BF16 && I % 8 == 0) {
      const int per_row = I / 8;
      const int vt = per_row >= 256 ? 256 : 64;
      hipLaunchKernelGGL(swiglu_vec8_kernel<ACT>, dim3((per_row + vt - 1) / vt, rows), dim3(vt), 0, stream,
                         (const bf16_t*)gate_up + (size_t)t0 * 2 * I, (bf16_t*)out + (size_t)t0 * I, I);
      continue;
    }
    Q3_DISPATCH_DTYPE(dtype, TT,
                      hipLaunchKernelGGL((swiglu_kernel<TT, ACT>), dim3((I + threads - 1) / threads, rows),
                                         dim3(threads), 0, stream,
                                         (const TT*)gate_up + (size_t)t0 * 2 * I, (TT*)out + (size_t)t0 * I, I));
  }
  return q3_launch_status();
}

// `act`: 0 silu, 1 the tanh form of gelu, 2 the exact gelu.
extern "C" int q3_gated_act(const void* gate_up, void* out, int T, int I, int act, int dtype, hipStream_t stream) {
  if (T <= 0 || I <= 0 || T > 65535 * 32 || act < 0 || act > 2) return Q3_ERR_BAD_ARGUMENT;
  if (act == 0) return launch_gated_act<0>(gate_up, out, T, I, dtype, stream);
  if (act == 1) return launch_gated_act<1>(gate_up, out, T, I, dtype, stream);
  return launch_gated_act<2>(gate_up, out, T, I, dtype, stream);
}

extern "C" int q3_swiglu(const void* gate_up, void* out, int T, int I, int dtype, hipStream_t stream) {
  return q3_gated_act(gate_up, out, T, I, 0, dtype, stream);
}

// out = gelu(x), elementwise in float32, rounded once: kind 0 the exact form
// 0.5 z (1 + erf(z / sqrt 2)), kind 1 the tanh form 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
__device__ inline float gelu_value(float z, int kind) {
  if (kind == 0) return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
  return 0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void gelu_kernel(const T* __restrict__ x, T* __restrict__ out, size_t n, int kind) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    out[i] = from_float<T>(gelu_value(to_float(x[i]), kind));
}

extern "C" int q3_gelu(const void* x, void* out, long n, int kind, int dtype, hipStream_t stream) {
  if (n <= 0 || kind < 0 || kind > 1) return Q3_ERR_BAD_ARGUMENT;
  long blocks = (n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  Q3_DISPATCH_DTYPE(dtype, TT, hipLaunchKernelGGL(gelu_kernel<TT>, dim3((unsigned)blocks), dim3(256), 0, stream,
                                                  (const TT*)x, (TT*)out, (size_t)n, kind));
  return q3_launch_status();
}
