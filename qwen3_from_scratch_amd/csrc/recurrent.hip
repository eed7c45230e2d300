// Mixers that carry a state of fixed size from token to token: a short causal convolution per
// channel, the Mamba-2 recurrence, the gates and the recurrence of Griffin's recurrent unit, and
// retention. A step's tokens are packed on one axis; sequence b owns rows cu[b] .. cu[b + 1] - 1
// and the state at row slots[b] of the state tensor (rows `state_stride` floats apart). States,
// decays, step sizes, gates and angles are float32.
#include "common.h"

#define Q3_TAPS_MOST 8

__device__ inline float softplus_value(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ inline float silu_value(float z) { return z / (1.f + expf(-z)); }
__device__ inline float sigmoid_value(float z) { return 1.f / (1.f + expf(-z)); }

// ---- causal convolution ----
// out[t, c] = act(bias[c] + sum_j w[c, taps - 1 - j] * in[t - j, c]), in = x (+ in_bias); inputs
// before the step's first row come from the state's tail ((taps - 1, C), oldest first), zeros at
// a sequence's start because a fresh state is zero.
template <typename TI, typename TO>
__global__ void causal_conv_kernel(const TI* __restrict__ x, long x_stride, const float* __restrict__ in_bias,
                                   const float* __restrict__ w, const float* __restrict__ bias,
                                   const float* __restrict__ state, long state_stride, const int* __restrict__ slots,
                                   const int* __restrict__ cu, const int* __restrict__ seq_index, TO* __restrict__ out,
                                   int C, int taps, int act) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = seq_index[t];
  const int start = cu[b];
  const float* tail = state + (size_t)slots[b] * state_stride;
  const float add = in_bias ? in_bias[c] : 0.f;
  float acc = bias[c];
  for (int j = 0; j < taps; ++j) {
    const int src = t - j;
    const float v = src >= start ? to_float(x[(size_t)src * x_stride + c]) + add
                                 : tail[(size_t)(taps - 1 - (start - src)) * C + c];
    acc += w[(size_t)c * taps + taps - 1 - j] * v;
  }
  if (act == 1) acc = silu_value(acc);
  out[(size_t)t * C + c] = from_float<TO>(acc);
}

// The tail after the step: the last taps - 1 inputs of the sequence, from this step's rows or,
// for a step shorter than that, from the old tail moved up.
template <typename TI>
__global__ void conv_tail_kernel(const TI* __restrict__ x, long x_stride, const float* __restrict__ in_bias,
                                 float* __restrict__ state, long state_stride, const int* __restrict__ slots,
                                 const int* __restrict__ cu, int C, int taps) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int start = cu[b], end = cu[b + 1];
  const int n = end - start;
  if (n <= 0) return;
  float* tail = state + (size_t)slots[b] * state_stride;
  const float add = in_bias ? in_bias[c] : 0.f;
  float keep[Q3_TAPS_MOST];
  for (int k = 0; k < taps - 1; ++k) {
    const int src = end - (taps - 1) + k;
    keep[k] = src >= start ? to_float(x[(size_t)src * x_stride + c]) + add : tail[(size_t)(k + n) * C + c];
  }
  for (int k = 0; k < taps - 1; ++k) tail[(size_t)k * C + c] = keep[k];
}

// ---- Mamba-2 ----
// One wavefront per (sequence, head, 64 columns of the head's vdim): lane p keeps column p of the
// state S (N x vdim) in registers and walks the sequence's tokens in order:
//   dt = softplus(dt_raw + dt_bias),  S = exp(-exp(A_log) dt) S + dt B x_p,  y_p = sum_n S[n] C[n] + D x_p.
// xbc rows are [x: H P | B: G N | C: G N]; B and C of the head's group go through shared memory.
template <typename TA, int NMAX>
__global__ void __launch_bounds__(64) mamba2_scan_kernel(
    const TA* __restrict__ xbc, const TA* __restrict__ dt, long dt_stride, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ state, long state_stride,
    const int* __restrict__ slots, const int* __restrict__ cu, float* __restrict__ y, int H, int P, int N, int G) {
  __shared__ float sB[NMAX], sC[NMAX];
  const int lane = threadIdx.x;
  const int p = blockIdx.x * 64 + lane;
  const int h = blockIdx.y, b = blockIdx.z;
  const int start = cu[b], end = cu[b + 1];
  if (end <= start) return;
  const int g = h / (H / G);
  const int C = H * P + 2 * G * N;
  const bool live = p < P;
  float* mine = state + (size_t)slots[b] * state_stride + (size_t)h * N * P + p;
  float S[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) S[n] = (live && n < N) ? mine[(size_t)n * P] : 0.f;
  const float rate = expf(a_log[h]), shift = dt_bias[h], skip = d_skip[h];
  for (int t = start; t < end; ++t) {
    const TA* row = xbc + (size_t)t * C;
    for (int n = lane; n < N; n += 64) {
      sB[n] = to_float(row[H * P + g * N + n]);
      sC[n] = to_float(row[H * P + G * N + g * N + n]);
    }
    __syncthreads();
    const float step = softplus_value(to_float(dt[(size_t)t * dt_stride + h]) + shift);
    const float decay = expf(-rate * step);
    const float xv = live ? to_float(row[h * P + p]) : 0.f;
    const float push = step * xv;
    float acc = 0.f;
#pragma unroll
    for (int n = 0; n < NMAX; ++n) {
      if (n < N) {
        S[n] = decay * S[n] + sB[n] * push;
        acc += S[n] * sC[n];
      }
    }
    if (live) y[(size_t)t * H * P + h * P + p] = acc + skip * xv;
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) mine[(size_t)n * P] = S[n];
  }
}

// ---- the recurrent unit's gates ----
// out[g, t, b * bw + o] = sigmoid(bias[g, b, o] + sum_i w[g, b, i, o] * u[t, b * bw + i]) for the
// two gates g, block-diagonal over `blocks` parts of bw numbers. A block of threads takes eight
// tokens of one part of one gate; their u lie in shared memory.
#define Q3_GATE_TOKENS 8
__global__ void block_gates_kernel(const float* __restrict__ u, const float* __restrict__ w,
                                   const float* __restrict__ bias, float* __restrict__ out, int T, int width, int bw) {
  extern __shared__ float su[];          // (Q3_GATE_TOKENS, bw)
  const int t0 = blockIdx.x * Q3_GATE_TOKENS;
  const int b = blockIdx.y, g = blockIdx.z;
  const int blocks = width / bw;
  for (int i = threadIdx.x; i < Q3_GATE_TOKENS * bw; i += blockDim.x) {
    const int tt = i / bw, e = i % bw;
    su[i] = t0 + tt < T ? u[(size_t)(t0 + tt) * width + b * bw + e] : 0.f;
  }
  __syncthreads();
  const float* wb = w + ((size_t)g * blocks + b) * bw * bw;
  for (int o = threadIdx.x; o < bw; o += blockDim.x) {
    float acc[Q3_GATE_TOKENS];
    const float start = bias[((size_t)g * blocks + b) * bw + o];
#pragma unroll
    for (int tt = 0; tt < Q3_GATE_TOKENS; ++tt) acc[tt] = start;
    for (int i = 0; i < bw; ++i) {
      const float wv = wb[(size_t)i * bw + o];
#pragma unroll
      for (int tt = 0; tt < Q3_GATE_TOKENS; ++tt) acc[tt] += wv * su[tt * bw + i];
    }
#pragma unroll
    for (int tt = 0; tt < Q3_GATE_TOKENS; ++tt)
      if (t0 + tt < T) out[((size_t)g * T + t0 + tt) * width + b * bw + o] = sigmoid_value(acc[tt]);
  }
}

// ---- the recurrent unit's recurrence ----
// Per (sequence, channel): log a = -rate r, a = exp(log a), S = a S + sqrt(1 - a^2) i u (1 - a^2 as
// -expm1(2 log a)), out = S * gelu_tanh(y + y_bias). gates = [r | i], each (T, width).
template <typename TO>
__global__ void rglru_scan_kernel(const float* __restrict__ u, const float* __restrict__ gates,
                                  const float* __restrict__ rate, const float* __restrict__ y, long y_stride,
                                  const float* __restrict__ y_bias, float* __restrict__ state, long state_stride,
                                  const int* __restrict__ slots, const int* __restrict__ cu, TO* __restrict__ out, int T,
                                  int width) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int b = blockIdx.y;
  if (c >= width) return;
  const int start = cu[b], end = cu[b + 1];
  if (end <= start) return;
  float* mine = state + (size_t)slots[b] * state_stride + c;
  float S = *mine;
  const float k = rate[c], yb = y_bias[c];
  for (int t = start; t < end; ++t) {
    const size_t at = (size_t)t * width + c;
    const float log_a = -k * gates[at];
    const float a = expf(log_a);
    S = a * S + sqrtf(-expm1f(2.f * log_a)) * gates[(size_t)T * width + at] * u[at];
    const float z = y[(size_t)t * y_stride + c] + yb;
    const float branch = 0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
    out[at] = from_float<TO>(S * branch);
  }
  *mine = S;
}

// ---- retention ----
// One block per (sequence, head), thread v keeps column v of S (dim x vdim) in registers. Rows of
// the input are [q: H dim | k: H dim | v: H vdim | g: H vdim]. Per token q and k turn by the
// position (pairs (i, i + half) of their first 2 * half numbers, angle = position * inv_freq[i]),
// k times k_scale; S = decay S + k v^T, o = S^T q; o is divided by the root mean square of the
// head's vdim numbers and multiplied by silu(g).
template <typename TA, int DMAX>
__global__ void retention_scan_kernel(const TA* __restrict__ rows, const float* __restrict__ inv_freq, int half,
                                      const int* __restrict__ positions, const float* __restrict__ decays, float k_scale,
                                      float eps, float* __restrict__ state, long state_stride,
                                      const int* __restrict__ slots, const int* __restrict__ cu, TA* __restrict__ out,
                                      int H, int dim, int vdim) {
  __shared__ float sq[DMAX], sk[DMAX];
  __shared__ float scratch[17];
  const int v = threadIdx.x;
  const int h = blockIdx.x, b = blockIdx.y;
  const int start = cu[b], end = cu[b + 1];
  if (end <= start) return;
  const bool live = v < vdim;
  const int hd = H * dim, hv = H * vdim;
  const size_t width = 2 * (size_t)hd + 2 * (size_t)hv;
  float* mine = state + (size_t)slots[b] * state_stride + (size_t)h * dim * vdim + v;
  float S[DMAX];
#pragma unroll
  for (int n = 0; n < DMAX; ++n) S[n] = (live && n < dim) ? mine[(size_t)n * vdim] : 0.f;
  const float decay = decays[h];
  for (int t = start; t < end; ++t) {
    const TA* row = rows + (size_t)t * width;
    const TA* q = row + h * dim;
    const TA* k = row + hd + h * dim;
    const float pos = (float)positions[t];
    for (int j = v; j < dim; j += blockDim.x) {
      float qv = to_float(q[j]), kv = to_float(k[j]);
      if (j < 2 * half) {
        const bool first = j < half;
        const int partner = first ? j + half : j - half;
        const float angle = pos * inv_freq[first ? j : j - half];
        const float c = cosf(angle), s = sinf(angle);
        const float qp = to_float(q[partner]), kp = to_float(k[partner]);
        qv = first ? qv * c - qp * s : qv * c + qp * s;
        kv = first ? kv * c - kp * s : kv * c + kp * s;
      }
      sq[j] = qv;
      sk[j] = kv * k_scale;
    }
    __syncthreads();
    const float vv = live ? to_float(row[2 * hd + h * vdim + v]) : 0.f;
    float acc = 0.f;
#pragma unroll
    for (int n = 0; n < DMAX; ++n) {
      if (n < dim) {
        S[n] = decay * S[n] + sk[n] * vv;
        acc += S[n] * sq[n];
      }
    }
    const float total = block_sum(live ? acc * acc : 0.f, scratch);
    if (live) {
      const float g = to_float(row[2 * hd + hv + h * vdim + v]);
      out[(size_t)t * hv + h * vdim + v] = from_float<TA>(acc * rsqrtf(total / (float)vdim + eps) * silu_value(g));
    }
  }
  if (live) {
#pragma unroll
    for (int n = 0; n < DMAX; ++n)
      if (n < dim) mine[(size_t)n * vdim] = S[n];
  }
}

// ---- launchers ----

extern "C" int q3_causal_conv(const void* x, long x_stride, const float* in_bias, const float* w, const float* bias,
                              float* state, long state_stride, const int* slots, const int* cu, const int* seq_index,
                              void* out, int T, int B, int C, int taps, int act, int in_dtype, int out_dtype,
                              hipStream_t stream) {
  if (T <= 0 || B <= 0 || C <= 0 || taps < 1 || taps > Q3_TAPS_MOST || act < 0 || act > 1) return Q3_ERR_BAD_ARGUMENT;
  const int threads = C >= 256 ? 256 : 64;
  const int chunks = (C + threads - 1) / threads;
  if (chunks > 65535) return Q3_ERR_UNSUPPORTED;
  Q3_DISPATCH_DTYPE(in_dtype, TI, Q3_DISPATCH_DTYPE(out_dtype, TO, {
                      hipLaunchKernelGGL((causal_conv_kernel<TI, TO>), dim3(T, chunks), dim3(threads), 0, stream,
                                         (const TI*)x, x_stride, in_bias, w, bias, state, state_stride, slots, cu,
                                         seq_index, (TO*)out, C, taps, act);
                    }));
  if (taps > 1)
    Q3_DISPATCH_DTYPE(in_dtype, TI,
                      hipLaunchKernelGGL(conv_tail_kernel<TI>, dim3(B, chunks), dim3(threads), 0, stream, (const TI*)x,
                                         x_stride, in_bias, state, state_stride, slots, cu, C, taps));
  return q3_launch_status();
}

template <typename TA>
static int launch_mamba2(const void* xbc, const void* dt, long dt_stride, const float* dt_bias, const float* a_log,
                         const float* d_skip, float* state, long state_stride, const int* slots, const int* cu, float* y,
                         int B, int H, int P, int N, int G, hipStream_t stream) {
  const dim3 grid((P + 63) / 64, H, B);
#define Q3_MAMBA(NMAX)                                                                                              \
  hipLaunchKernelGGL((mamba2_scan_kernel<TA, NMAX>), grid, dim3(64), 0, stream, (const TA*)xbc, (const TA*)dt,      \
                     dt_stride, dt_bias, a_log, d_skip, state, state_stride, slots, cu, y, H, P, N, G)
  if (N <= 16) Q3_MAMBA(16);
  else if (N <= 32) Q3_MAMBA(32);
  else if (N <= 64) Q3_MAMBA(64);
  else if (N <= 128) Q3_MAMBA(128);
  else Q3_MAMBA(256);
#undef Q3_MAMBA
  return q3_launch_status();
}

extern "C" int q3_mamba2_scan(const void* xbc, const void* dt, long dt_stride, const float* dt_bias, const float* a_log,
                              const float* d_skip, float* state, long state_stride, const int* slots, const int* cu,
                              float* y, int B, int H, int P, int N, int G, int act_dtype, hipStream_t stream) {
  if (B <= 0 || H <= 0 || P <= 0 || N <= 0 || G <= 0 || H % G || H > 65535 || B > 65535) return Q3_ERR_BAD_ARGUMENT;
  if (N > 256) return Q3_ERR_UNSUPPORTED;
  Q3_DISPATCH_DTYPE(act_dtype, TA, return launch_mamba2<TA>(xbc, dt, dt_stride, dt_bias, a_log, d_skip, state,
                                                            state_stride, slots, cu, y, B, H, P, N, G, stream));
  return 0;
}

extern "C" int q3_block_gates(const float* u, const float* w, const float* bias, float* out, int T, int width, int blocks,
                              hipStream_t stream) {
  if (T <= 0 || width <= 0 || blocks <= 0 || width % blocks || blocks > 65535) return Q3_ERR_BAD_ARGUMENT;
  const int bw = width / blocks;
  if (bw > 1536) return Q3_ERR_UNSUPPORTED;
  const int threads = bw >= 256 ? 256 : (bw >= 128 ? 128 : 64);
  hipLaunchKernelGGL(block_gates_kernel, dim3((T + Q3_GATE_TOKENS - 1) / Q3_GATE_TOKENS, blocks, 2), dim3(threads),
                     (size_t)Q3_GATE_TOKENS * bw * sizeof(float), stream, u, w, bias, out, T, width, bw);
  return q3_launch_status();
}

extern "C" int q3_rglru_scan(const float* u, const float* gates, const float* rate, const float* y, long y_stride,
                             const float* y_bias, float* state, long state_stride, const int* slots, const int* cu,
                             void* out, int T, int B, int width, int out_dtype, hipStream_t stream) {
  if (T <= 0 || B <= 0 || width <= 0 || B > 65535) return Q3_ERR_BAD_ARGUMENT;
  const int threads = width >= 256 ? 256 : 64;
  Q3_DISPATCH_DTYPE(out_dtype, TO,
                    hipLaunchKernelGGL(rglru_scan_kernel<TO>, dim3((width + threads - 1) / threads, B), dim3(threads), 0,
                                       stream, u, gates, rate, y, y_stride, y_bias, state, state_stride, slots, cu,
                                       (TO*)out, T, width));
  return q3_launch_status();
}

template <typename TA>
static int launch_retention(const void* rows, const float* inv_freq, int half, const int* positions, const float* decays,
                            float k_scale, float eps, float* state, long state_stride, const int* slots, const int* cu,
                            void* out, int B, int H, int dim, int vdim, hipStream_t stream) {
  const dim3 grid(H, B);
  const dim3 block((vdim + 63) / 64 * 64);
#define Q3_RETENTION(DMAX)                                                                                          \
  hipLaunchKernelGGL((retention_scan_kernel<TA, DMAX>), grid, block, 0, stream, (const TA*)rows, inv_freq, half,   \
                     positions, decays, k_scale, eps, state, state_stride, slots, cu, (TA*)out, H, dim, vdim)
  if (dim <= 32) Q3_RETENTION(32);
  else if (dim <= 64) Q3_RETENTION(64);
  else if (dim <= 128) Q3_RETENTION(128);
  else Q3_RETENTION(256);
#undef Q3_RETENTION
  return q3_launch_status();
}

extern "C" int q3_retention_scan(const void* rows, const float* inv_freq, int half, const int* positions,
                                 const float* decays, float k_scale, float eps, float* state, long state_stride,
                                 const int* slots, const int* cu, void* out, int B, int H, int dim, int vdim,
                                 int act_dtype, hipStream_t stream) {
  if (B <= 0 || H <= 0 || dim <= 0 || vdim <= 0 || half < 0 || 2 * half > dim || H > 65535 || B > 65535)
    return Q3_ERR_BAD_ARGUMENT;
  if (half > 0 && !inv_freq) return Q3_ERR_BAD_ARGUMENT;
  if (dim > 256 || vdim > 1024) return Q3_ERR_UNSUPPORTED;
  Q3_DISPATCH_DTYPE(act_dtype, TA, return launch_retention<TA>(rows, inv_freq, half, positions, decays, k_scale, eps,
                                                               state, state_stride, slots, cu, out, B, H, dim, vdim,
                                                               stream));
  return 0;
}
