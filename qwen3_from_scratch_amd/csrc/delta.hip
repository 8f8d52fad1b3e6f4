// The gated delta rule with one decay per head and key channel. Per head, with S (dim x vdim)
// carried from token to token in float32:
//
//   S <- diag(g_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
//
// so the read-out sees the current token's write. q and k are unit vectors per head (q also times
// dim^(-1/2)), g = exp(-exp(a_log) softplus(a + dt_bias)), beta = sigmoid(b). Every column of S is
// a recurrence of its own (a column's u, its update and its read-out touch no other column), so
// the columns are shared out over the chip: sixteen lanes hold one column, a lane `R` consecutive
// rows of it, and the two sums over the rows are sums over a row of sixteen lanes.
//
// A step's tokens are packed on one axis; sequence b owns rows cu[b] .. cu[b + 1] - 1 and the state
// at row slots[b] of the state tensor (rows `state_stride` floats apart), laid out (head, vdim, dim):
// a column's numbers side by side. Unit norms, decays, step sizes, gates and S are float32.
#include "common.h"

__device__ inline float delta_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ inline float delta_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }

// ---- what the recurrence reads, per token ----
// One block per token. `conv` float32 (T, 2 G dim + H vdim): [q | k | v] behind their convolutions
// and activations. `b_logits` (T, H) and `a_logits` (T, H dim), float32 rows possibly apart. Writes
// `packed` (T, H, 3, DP) float32, per head [k | q | g], each padded with zeros to DP numbers (a
// padded row of S then stays zero), q and k as unit vectors per head: x / sqrt(sum(x^2) + unit_eps),
// q times dim^(-1/2), head h taking q and k of group h / (H / G); and `beta` (T, H, 2): beta itself and
// the head's k . q, which the recurrence uses to read the current token's write without waiting for it.
__global__ void __launch_bounds__(256) delta_prepare_kernel(
    const float* __restrict__ conv, const float* __restrict__ b_logits, long b_stride, const float* __restrict__ a_logits,
    long a_stride, const float* __restrict__ dt_bias, const float* __restrict__ a_log, float unit_eps,
    float* __restrict__ packed, float* __restrict__ beta, int H, int G, int dim, int vdim, int DP) {
  extern __shared__ float unit[];             // (2, G, dim): q then k, finished; then (G): k . q
  const int t = blockIdx.x;
  const int wave = threadIdx.x / Q3_WAVE, lane = threadIdx.x % Q3_WAVE, waves = blockDim.x / Q3_WAVE;
  const int C = 2 * G * dim + H * vdim;
  const float* row = conv + (size_t)t * C;
  for (int j = wave; j < 2 * G; j += waves) {           // j < G: a head of q, else a head of k
    const float* src = row + (size_t)j * dim;
    float acc = 0.f;
    for (int e = lane; e < dim; e += Q3_WAVE) acc += src[e] * src[e];
    float r = rsqrtf(wave_sum(acc) + unit_eps);
    if (j < G) r *= rsqrtf((float)dim);
    for (int e = lane; e < dim; e += Q3_WAVE) unit[j * dim + e] = src[e] * r;
  }
  __syncthreads();
  float* kq = unit + 2 * G * dim;
  for (int j = wave; j < G; j += waves) {
    float acc = 0.f;
    for (int e = lane; e < dim; e += Q3_WAVE) acc += unit[j * dim + e] * unit[(G + j) * dim + e];
    acc = wave_sum(acc);
    if (lane == 0) kq[j] = acc;
  }
  __syncthreads();
  const int per = H / G;
  for (int i = threadIdx.x; i < H * DP; i += blockDim.x) {
    const int h = i / DP, e = i - h * DP;
    float* dst = packed + ((size_t)t * H + h) * 3 * DP;
    float k = 0.f, q = 0.f, g = 0.f;
    if (e < dim) {
      const int grp = h / per;
      q = unit[grp * dim + e];
      k = unit[(G + grp) * dim + e];
      const float step = delta_softplus(a_logits[(size_t)t * a_stride + h * dim + e] + dt_bias[h * dim + e]);
      g = expf(-expf(a_log[h]) * step);
    }
    dst[e] = k;
    dst[DP + e] = q;
    dst[2 * DP + e] = g;
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    beta[((size_t)t * H + h) * 2] = delta_sigmoid(b_logits[(size_t)t * b_stride + h]);
    beta[((size_t)t * H + h) * 2 + 1] = kq[h / per];
  }
}

// ---- the recurrence ----
template <int CTRL>
__device__ __forceinline__ float lanes_moved(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int R>
__device__ __forceinline__ void load_run(const float* p, float (&v)[R]) {
  if constexpr (R >= 4) {
#pragma unroll
    for (int j = 0; j < R / 4; ++j) {
      const float4 a = *reinterpret_cast<const float4*>(p + 4 * j);
      v[4 * j] = a.x, v[4 * j + 1] = a.y, v[4 * j + 2] = a.z, v[4 * j + 3] = a.w;
    }
  } else {
    const float2 a = *reinterpret_cast<const float2*>(p);
    v[0] = a.x, v[1] = a.y;
  }
}

#define Q3_DELTA_COLS 16       // columns of S a block of 256 threads holds
// grid (H * ceil(vdim / 16), B), 256 threads: thread (column slot = t / 16, part = t % 16) keeps rows
// part * R .. part * R + R - 1 of its column in registers. The tokens' [k | q | g] come `TC` tokens at
// a time through shared memory, the next chunk's on their way (into registers) while this one is worked
// on, and within a chunk the next token's numbers are read from shared memory while this token's are
// worked on. A token's chain of dependent steps is what bounds the kernel (one wavefront a SIMD when a
// single sequence is all there is), so the read-out does not wait for the write: with S' = diag(g) S,
//   u = beta (v - S'^T k),   o = (S' + k u^T)^T q = S'^T q + u (k . q),
// the two sums over the rows run side by side, k . q comes with the token, and the update S = S' + k u^T
// is off the way to o. The order of a column's arithmetic does not depend on how the sequence was cut
// into steps or chunks. Results go to `raw` (T, H vdim) float32; the division by the head's root mean
// square and the gate follow in delta_finish_kernel.
template <int R>
struct DeltaToken {
  float k[R], q[R], g[R], v, beta, kq;
};

template <int R, int TC>
__global__ void __launch_bounds__(256) delta_scan_kernel(
    const float* __restrict__ packed, const float* __restrict__ beta, const float* __restrict__ conv,
    float* __restrict__ state, long state_stride, const int* __restrict__ slots, const int* __restrict__ cu,
    float* __restrict__ raw, int H, int G, int dim, int vdim) {
  constexpr int DP = 16 * R;
  constexpr int ROW = 3 * DP;                       // floats of one token's [k | q | g]
  constexpr int N4 = TC * ROW / 4;                  // 16-byte pieces of a chunk
  constexpr int PF = (N4 + 255) / 256;              // pieces a thread brings
  __shared__ __attribute__((aligned(16))) float kqg[2][TC * ROW];
  __shared__ float sv[2][TC * Q3_DELTA_COLS];
  __shared__ __attribute__((aligned(8))) float sb[2][2 * TC];
  const int slices = (vdim + Q3_DELTA_COLS - 1) / Q3_DELTA_COLS;
  const int h = blockIdx.x / slices, c0 = (blockIdx.x % slices) * Q3_DELTA_COLS;
  const int b = blockIdx.y;
  const int start = cu[b], end = cu[b + 1];
  if (end <= start) return;
  const int tid = threadIdx.x;
  const int slot = tid >> 4, part = tid & 15;
  const int c = c0 + slot;
  const bool live = c < vdim;
  const int C = 2 * G * dim + H * vdim;
  const int v_at = 2 * G * dim + h * vdim;

  float* mine = state + (size_t)slots[b] * state_stride + ((size_t)h * vdim + (live ? c : 0)) * dim + part * R;
  float S[R];
  // a thread's rows lie side by side in the state: 16-byte accesses where the column's start allows them
  const bool whole = live && part * R + R <= dim && R >= 4 && ((size_t)mine % 16) == 0;
  if (whole) {
    load_run<R>(mine, S);
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r) S[r] = (live && part * R + r < dim) ? mine[r] : 0.f;
  }

  float4 ahead[PF];
  float ahead_v = 0.f, ahead_b = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int at = tid + 256 * i;                 // piece `at` of the chunk: token at / (ROW / 4)
      const int tok = at / (ROW / 4), off = at - tok * (ROW / 4);
      ahead[i] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (at < N4 && t0 + tok < end)
        ahead[i] = *reinterpret_cast<const float4*>(packed + ((size_t)(t0 + tok) * H + h) * ROW + 4 * off);
    }
    if (tid < TC * Q3_DELTA_COLS) {
      const int tok = tid >> 4, col = c0 + (tid & 15);
      ahead_v = (t0 + tok < end && col < vdim) ? conv[(size_t)(t0 + tok) * C + v_at + col] : 0.f;
    }
    if (tid < 2 * TC) ahead_b = t0 + (tid >> 1) < end ? beta[((size_t)(t0 + (tid >> 1)) * H + h) * 2 + (tid & 1)] : 0.f;
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int at = tid + 256 * i;
      if (at < N4) *reinterpret_cast<float4*>(&kqg[buf][4 * at]) = ahead[i];
    }
    if (tid < TC * Q3_DELTA_COLS) sv[buf][tid] = ahead_v;
    if (tid < 2 * TC) sb[buf][tid] = ahead_b;
  };
  auto read = [&](DeltaToken<R>& tok, int buf, int i) {      // token i of the chunk in `buf`, from shared memory
    const float* row = &kqg[buf][i * ROW + part * R];
    load_run<R>(row, tok.k);
    load_run<R>(row + 2 * DP, tok.g);
    load_run<R>(row + DP, tok.q);
    tok.v = sv[buf][i * Q3_DELTA_COLS + slot];
    const float2 bk = *reinterpret_cast<const float2*>(&sb[buf][2 * i]);
    tok.beta = bk.x;
    tok.kq = bk.y;
  };
  auto work = [&](const DeltaToken<R>& tok, int t) {
    float seen[2] = {0.f, 0.f}, out[2] = {0.f, 0.f};
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] *= tok.g[r];
      seen[r & 1] += S[r] * tok.k[r];
      out[r & 1] += S[r] * tok.q[r];
    }
    float a = seen[0] + seen[1], o = out[0] + out[1];
    a += lanes_moved<0xB1>(a);      // quad_perm [1, 0, 3, 2]: the two sums over sixteen lanes, step by step side by side
    o += lanes_moved<0xB1>(o);
    a += lanes_moved<0x4E>(a);      // quad_perm [2, 3, 0, 1]
    o += lanes_moved<0x4E>(o);
    a += lanes_moved<0x124>(a);     // row_ror 4
    o += lanes_moved<0x124>(o);
    a += lanes_moved<0x128>(a);     // row_ror 8
    o += lanes_moved<0x128>(o);
    const float u = tok.beta * (tok.v - a);
#pragma unroll
    for (int r = 0; r < R; ++r) S[r] += tok.k[r] * u;
    if (part == 0 && live) raw[(size_t)t * H * vdim + (size_t)h * vdim + c] = o + u * tok.kq;
  };

  fetch(start);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int t0 = start; t0 < end; t0 += TC, buf ^= 1) {
    const bool more = t0 + TC < end;                // uniform in the block
    if (more) fetch(t0 + TC);
    const int n = end - t0 < TC ? end - t0 : TC;
    // two tokens in work while the next two come from shared memory
    DeltaToken<R> a0, a1, b0, b1;
    auto at = [&](int i) { return i < TC ? i : TC - 1; };
    read(a0, buf, 0);
    read(a1, buf, at(1));
    for (int i = 0; i < n; i += 4) {
      read(b0, buf, at(i + 2));
      read(b1, buf, at(i + 3));
      work(a0, t0 + i);
      if (i + 1 < n) work(a1, t0 + i + 1);
      if (i + 2 < n) {
        read(a0, buf, at(i + 4));
        read(a1, buf, at(i + 5));
        work(b0, t0 + i + 2);
        if (i + 3 < n) work(b1, t0 + i + 3);
      }
    }
    if (more) put(buf ^ 1);
    __syncthreads();
  }
  if (whole) {
    if constexpr (R >= 4) {
#pragma unroll
      for (int j = 0; j < R / 4; ++j)
        *reinterpret_cast<float4*>(mine + 4 * j) = make_float4(S[4 * j], S[4 * j + 1], S[4 * j + 2], S[4 * j + 3]);
    }
  } else if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (part * R + r < dim) mine[r] = S[r];
  }
}

// ---- behind the recurrence ----
// grid (T, H): out[t, h, :] = o / sqrt(mean(o^2) + eps) * weight * sigmoid(gate[t, h, :]), o = raw[t, h, :],
// `weight` vdim numbers that all heads share, `gate` float32 (T, H vdim) rows possibly apart.
template <typename TA>
__global__ void delta_finish_kernel(const float* __restrict__ raw, const float* __restrict__ gate, long gate_stride,
                                    const float* __restrict__ weight, float eps, TA* __restrict__ out, int H, int vdim) {
  __shared__ float scratch[17];
  const int t = blockIdx.x, h = blockIdx.y;
  const float* o = raw + ((size_t)t * H + h) * vdim;
  float acc = 0.f;
  for (int e = threadIdx.x; e < vdim; e += blockDim.x) acc += o[e] * o[e];
  const float r = rsqrtf(block_sum(acc, scratch) / (float)vdim + eps);
  for (int e = threadIdx.x; e < vdim; e += blockDim.x)
    out[((size_t)t * H + h) * vdim + e] =
        from_float<TA>(o[e] * r * weight[e] * delta_sigmoid(gate[(size_t)t * gate_stride + h * vdim + e]));
}

// The padded key size the recurrence works with, and the floats of scratch a step of T tokens needs:
// packed (T, H, 3, DP), beta (T, H, 2), raw (T, H vdim).
extern "C" int q3_channel_delta_padded(int dim) {
  return dim <= 32 ? 32 : (dim <= 64 ? 64 : (dim <= 128 ? 128 : 256));
}
extern "C" long q3_channel_delta_workspace(int T, int H, int dim, int vdim) {
  return (long)T * H * (3 * q3_channel_delta_padded(dim) + 2 + vdim);
}

// conv float32 (T, 2 G dim + H vdim) contiguous; b_logits (T, H), a_logits (T, H dim) and gate (T, H vdim)
// float32 with their rows' strides; dt_bias (H dim), a_log (H), norm_weight (vdim) float32; state rows hold
// (H, vdim, dim); out (T, H vdim) of `act_dtype`; `work`: q3_channel_delta_workspace floats, 16-byte aligned.
extern "C" int q3_channel_delta(const float* conv, const float* b_logits, long b_stride, const float* a_logits,
                                long a_stride, const float* gate, long gate_stride, const float* dt_bias,
                                const float* a_log, const float* norm_weight, float eps, float unit_eps, float* state,
                                long state_stride, const int* slots, const int* cu, void* out, float* work, int T, int B,
                                int H, int G, int dim, int vdim, int act_dtype, hipStream_t stream) {
  if (T <= 0 || B <= 0 || H <= 0 || G <= 0 || H % G || dim <= 0 || vdim <= 0 || B > 65535 || !work || ((size_t)work % 16))
    return Q3_ERR_BAD_ARGUMENT;
  const int slices = (vdim + Q3_DELTA_COLS - 1) / Q3_DELTA_COLS;
  if (dim > 256 || H > 65535 || (long)H * slices > 2147483647L || 2L * G * dim * sizeof(float) > 65536)
    return Q3_ERR_UNSUPPORTED;
  const int DP = q3_channel_delta_padded(dim);
  float* packed = work;
  float* beta = packed + (size_t)T * H * 3 * DP;
  float* raw = beta + (size_t)T * H * 2;
  hipLaunchKernelGGL(delta_prepare_kernel, dim3(T), dim3(256), ((size_t)2 * G * dim + G) * sizeof(float), stream, conv, b_logits,
                     b_stride, a_logits, a_stride, dt_bias, a_log, unit_eps, packed, beta, H, G, dim, vdim, DP);
  const dim3 grid(H * slices, B);
#define Q3_DELTA(RR, TT)                                                                                             \
  hipLaunchKernelGGL((delta_scan_kernel<RR, TT>), grid, dim3(256), 0, stream, packed, beta, conv, state, state_stride, \
                     slots, cu, raw, H, G, dim, vdim)
  // steps of a token or two a sequence (decoding): chunks of two tokens, whose few kilobytes of shared memory let
  // a CU hold as many blocks as its threads allow, where the wait for each block's state is what counts
  const bool few = T <= 2 * B;
  if (DP == 32) { if (few) Q3_DELTA(2, 2); else Q3_DELTA(2, 16); }
  else if (DP == 64) { if (few) Q3_DELTA(4, 2); else Q3_DELTA(4, 16); }
  else if (DP == 128) { if (few) Q3_DELTA(8, 2); else Q3_DELTA(8, 16); }
  else { if (few) Q3_DELTA(16, 2); else Q3_DELTA(16, 8); }
#undef Q3_DELTA
  const int threads = vdim >= 256 ? 256 : (vdim >= 128 ? 128 : 64);
  Q3_DISPATCH_DTYPE(act_dtype, TA, hipLaunchKernelGGL(delta_finish_kernel<TA>, dim3(T, H), dim3(threads), 0, stream, raw,
                                                      gate, gate_stride, norm_weight, eps, (TA*)out, H, vdim));
  return q3_launch_status();
}
