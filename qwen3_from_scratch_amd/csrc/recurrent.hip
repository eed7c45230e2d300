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
                                   const float* state, long state_stride, const int* __restrict__ slots,
                                   const int* __restrict__ cu, const int* __restrict__ seq_index, TO* __restrict__ out,
                                   int T, int C, int taps, int act, int rows_each, float* new_tail) {
  // a thread takes one channel of `rows_each` rows in a row: its taps and biases stay in registers.
  // `new_tail` (the state again, given only when every sequence brings one row): the thread then
  // also moves its sequence's tail up by that row, which nobody else reads in this step.
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const float add = in_bias ? in_bias[c] : 0.f;
  const float base = bias[c];
  float tap[Q3_TAPS_MOST];
#pragma unroll
  for (int j = 0; j < Q3_TAPS_MOST; ++j) tap[j] = j < taps ? w[(size_t)c * taps + taps - 1 - j] : 0.f;
  const int t0 = blockIdx.x * rows_each;
  const int t1 = t0 + rows_each < T ? t0 + rows_each : T;
  for (int t = t0; t < t1; ++t) {
    const int b = seq_index[t];
    const int start = cu[b];
    const float* tail = state + (size_t)slots[b] * state_stride;
    float acc = base;
#pragma unroll
    for (int j = 0; j < Q3_TAPS_MOST; ++j) {
      if (j < taps) {
        const int src = t - j;
        const float v = src >= start ? to_float(x[(size_t)src * x_stride + c]) + add
                                     : tail[(size_t)(taps - 1 - (start - src)) * C + c];
        acc += tap[j] * v;
      }
    }
    if (act == 1) acc = silu_value(acc);
    out[(size_t)t * C + c] = from_float<TO>(acc);
    if (new_tail) {
      float* mine = new_tail + (size_t)slots[b] * state_stride;
      float keep[Q3_TAPS_MOST];
#pragma unroll
      for (int k = 0; k < Q3_TAPS_MOST; ++k)
        if (k < taps - 1) keep[k] = k + 1 < taps - 1 ? mine[(size_t)(k + 1) * C + c] : to_float(x[(size_t)t * x_stride + c]) + add;
#pragma unroll
      for (int k = 0; k < Q3_TAPS_MOST; ++k)
        if (k < taps - 1) mine[(size_t)k * C + c] = keep[k];
    }
  }
}

// Eight channels a thread in 16-byte accesses, for steps of many rows: the thread walks `rows_each`
// rows with its last taps - 1 inputs in registers, so every input is read once; where a row is a
// sequence's first (or the thread's first), the inputs before it come from the rows above or from
// the sequence's tail. Needs C and the rows' stride in steps of eight and 16-byte aligned rows.
__device__ inline void load8(const bf16_t* p, float (&v)[8]) {
  union {
    uint4 u;
    bf16_t e[8];
  } a;
  a.u = *reinterpret_cast<const uint4*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = bf16_to_float(a.e[i]);
}
__device__ inline void load8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
}
__device__ inline void store8(bf16_t* p, const float (&v)[8]) {
  union {
    uint4 u;
    bf16_t e[8];
  } a;
#pragma unroll
  for (int i = 0; i < 8; ++i) a.e[i] = float_to_bf16(v[i]);
  *reinterpret_cast<uint4*>(p) = a.u;
}
__device__ inline void store8(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}

#define Q3_CONV_TILE 8
template <typename TI, typename TO>
__global__ void __launch_bounds__(64) causal_conv_wide_kernel(const TI* __restrict__ x, long x_stride, const float* __restrict__ in_bias,
                                        const float* __restrict__ w, const float* __restrict__ bias,
                                        const float* __restrict__ state, long state_stride,
                                        const int* __restrict__ slots, const int* __restrict__ cu,
                                        const int* __restrict__ seq_index, TO* __restrict__ out, int T, int C, int taps,
                                        int act, int rows_each) {
  // the block's taps lie side by side in memory (64 threads x 8 channels x taps): in through shared memory
  __shared__ __attribute__((aligned(16))) float taps_of_block[64 * 8 * Q3_TAPS_MOST];
  const int first = blockIdx.y * 64 * 8;
  const int held = C - first < 64 * 8 ? C - first : 64 * 8;
  {
    // 2 * taps loads of 16 bytes a thread, all asked for before the first is stored
    const float4* src = reinterpret_cast<const float4*>(w + (size_t)first * taps);
    const int pieces = held * taps / 4;
    float4 got[2 * Q3_TAPS_MOST];
#pragma unroll
    for (int k = 0; k < 2 * Q3_TAPS_MOST; ++k)
      got[k] = (k < 2 * taps && threadIdx.x + 64 * k < pieces) ? src[threadIdx.x + 64 * k] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int k = 0; k < 2 * Q3_TAPS_MOST; ++k)
      if (k < 2 * taps && threadIdx.x + 64 * k < pieces) reinterpret_cast<float4*>(taps_of_block)[threadIdx.x + 64 * k] = got[k];
  }
  __syncthreads();
  const int c0 = first + threadIdx.x * 8;
  if (c0 >= C) return;
  float tap[Q3_TAPS_MOST][8], base[8], add[8], win[Q3_TAPS_MOST - 1][8];
  load8(bias + c0, base);
#pragma unroll
  for (int e = 0; e < 8; ++e) add[e] = 0.f;
  if (in_bias) load8(in_bias + c0, add);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int j = 0; j < Q3_TAPS_MOST; ++j)
      tap[j][e] = j < taps ? taps_of_block[(threadIdx.x * 8 + e) * taps + taps - 1 - j] : 0.f;
  }
  const int t0 = blockIdx.x * rows_each;
  const int t1 = t0 + rows_each < T ? t0 + rows_each : T;
  if (rows_each == Q3_CONV_TILE && seq_index[t0] == seq_index[t1 - 1]) {
    // the usual case, all rows of one sequence: every input the rows need is asked for at once (one wait
    // instead of a chain of them), rows t0 - (taps - 1) .. t1 - 1 at in[Q3_TAPS_MOST - taps ..]
    const int b = seq_index[t0];
    const int start = cu[b];
    const float* tail = state + (size_t)slots[b] * state_stride;
    float in[Q3_CONV_TILE + Q3_TAPS_MOST - 1][8];
#pragma unroll
    for (int i = 0; i < Q3_CONV_TILE + Q3_TAPS_MOST - 1; ++i) {
      const int row = t0 - (Q3_TAPS_MOST - 1) + i;
      if (i >= Q3_TAPS_MOST - taps && row < t1) {
        if (row >= start) {
          load8(x + (size_t)row * x_stride + c0, in[i]);
#pragma unroll
          for (int e = 0; e < 8; ++e) in[i][e] += add[e];
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) in[i][e] = tail[(size_t)(taps - 1 - (start - row)) * C + c0 + e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) in[i][e] = 0.f;
      }
    }
#pragma unroll
    for (int r = 0; r < Q3_CONV_TILE; ++r) {
      if (t0 + r < t1) {
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = base[e];
#pragma unroll
        for (int j = 0; j < Q3_TAPS_MOST; ++j)
          if (j < taps) {
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += tap[j][e] * in[r + Q3_TAPS_MOST - 1 - j][e];
          }
        if (act == 1) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] = silu_value(acc[e]);
        }
        store8(out + (size_t)(t0 + r) * C + c0, acc);
      }
    }
    return;
  }
  for (int t = t0; t < t1; ++t) {
    const int b = seq_index[t];
    const int start = cu[b];
    if (t == t0 || t == start) {
      const float* tail = state + (size_t)slots[b] * state_stride;
#pragma unroll
      for (int j = 0; j < Q3_TAPS_MOST - 1; ++j) {
        if (j < taps - 1) {
          const int src = t - 1 - j;
          if (src >= start) {
            load8(x + (size_t)src * x_stride + c0, win[j]);
#pragma unroll
            for (int e = 0; e < 8; ++e) win[j][e] += add[e];
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) win[j][e] = tail[(size_t)(taps - 1 - (start - src)) * C + c0 + e];
          }
        }
      }
    }
    float cur[8], acc[8];
    load8(x + (size_t)t * x_stride + c0, cur);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      cur[e] += add[e];
      acc[e] = base[e] + tap[0][e] * cur[e];
    }
#pragma unroll
    for (int j = 0; j < Q3_TAPS_MOST - 1; ++j)
      if (j < taps - 1) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += tap[j + 1][e] * win[j][e];
      }
    if (act == 1) {
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = silu_value(acc[e]);
    }
    store8(out + (size_t)t * C + c0, acc);
#pragma unroll
    for (int j = Q3_TAPS_MOST - 2; j > 0; --j) {
#pragma unroll
      for (int e = 0; e < 8; ++e) win[j][e] = win[j - 1][e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) win[0][e] = cur[e];
  }
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
// two gates g, block-diagonal over `blocks` parts of bw numbers. A block of threads forms 64 tokens
// by 64 outputs of one part and gate, over the inputs in slices of 64 that go through shared
// memory (asked for in batches, as everywhere here); a thread holds 4 x 4 of them.
#define Q3_GATE_TOKENS 8
__global__ void __launch_bounds__(256) block_gates_kernel(const float* __restrict__ u, const float* __restrict__ w,
                                                          const float* __restrict__ bias, float* __restrict__ out, int T,
                                                          int width, int bw, int out_tiles) {
  __shared__ float one[64 * 65];           // (token, input), rows padded
  __shared__ __attribute__((aligned(16))) float two[64 * 64];           // (input, output)
  const int t0 = blockIdx.x * 64;
  const int b = blockIdx.y / out_tiles, o0 = (blockIdx.y % out_tiles) * 64, g = blockIdx.z;
  const int blocks = width / bw;
  const float* wb = w + ((size_t)g * blocks + b) * bw * bw;
  const int tt = threadIdx.x / 16, tj = threadIdx.x % 16;      // tokens tt + 16 r, outputs 4 tj .. 4 tj + 3
  float acc[4][4];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int x = 0; x < 4; ++x) acc[r][x] = 0.f;
  for (int i0 = 0; i0 < bw; i0 += 64) {
    __syncthreads();
    {
      float gu[16], gw[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const int e = threadIdx.x + 256 * k;
        const int s = e / 64, c = e % 64;
        gu[k] = (t0 + s < T && i0 + c < bw) ? u[(size_t)(t0 + s) * width + b * bw + i0 + c] : 0.f;
        gw[k] = (i0 + s < bw && o0 + c < bw) ? wb[(size_t)(i0 + s) * bw + o0 + c] : 0.f;
      }
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const int e = threadIdx.x + 256 * k;
        one[(e / 64) * 65 + e % 64] = gu[k];
        two[e] = gw[k];
      }
    }
    __syncthreads();
    for (int i = 0; i < 64; ++i) {
      const float4 wv = *reinterpret_cast<const float4*>(two + i * 64 + 4 * tj);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float uv = one[(tt + 16 * r) * 65 + i];
        acc[r][0] += uv * wv.x;
        acc[r][1] += uv * wv.y;
        acc[r][2] += uv * wv.z;
        acc[r][3] += uv * wv.w;
      }
    }
  }
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int o = o0 + 4 * tj + x;
    if (o < bw) {
      const float start = bias[((size_t)g * blocks + b) * bw + o];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = t0 + tt + 16 * r;
        if (t < T) out[((size_t)g * T + t) * width + b * bw + o] = sigmoid_value(start + acc[r][x]);
      }
    }
  }
}

// The same for steps of few rows, where the kernel above leaves most of the chip idle: a block
// takes 64 outputs of one part and gate for eight tokens, its four quarters of threads each a
// quarter of the inputs; the quarters' sums meet in shared memory in a fixed order.
__global__ void __launch_bounds__(256) block_gates_few_kernel(const float* __restrict__ u, const float* __restrict__ w,
                                                              const float* __restrict__ bias, float* __restrict__ out,
                                                              int T, int width, int bw, int out_tiles) {
  extern __shared__ float su[];          // (Q3_GATE_TOKENS, bw), then (4, 64, Q3_GATE_TOKENS) partial sums
  float* part = su + Q3_GATE_TOKENS * bw;
  const int t0 = blockIdx.x * Q3_GATE_TOKENS;
  const int b = blockIdx.y / out_tiles, tile = blockIdx.y % out_tiles, g = blockIdx.z;
  const int blocks = width / bw;
  for (int i = threadIdx.x; i < Q3_GATE_TOKENS * bw; i += 256) {
    const int tt = i / bw, e = i % bw;
    su[i] = t0 + tt < T ? u[(size_t)(t0 + tt) * width + b * bw + e] : 0.f;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, quarter = threadIdx.x >> 6;
  const int o = tile * 64 + lane;
  const int each = (bw + 3) / 4;
  const int i0 = quarter * each, i1 = i0 + each < bw ? i0 + each : bw;
  float acc[Q3_GATE_TOKENS];
#pragma unroll
  for (int tt = 0; tt < Q3_GATE_TOKENS; ++tt) acc[tt] = 0.f;
  if (o < bw) {
    const float* wb = w + ((size_t)g * blocks + b) * bw * bw + o;
    // eight weights at a time, all asked for before any is used: the loop is a chain of memory round trips otherwise
    for (int i = i0; i < i1; i += 8) {
      float wv[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) wv[j] = i + j < i1 ? wb[(size_t)(i + j) * bw] : 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int at = i + j < i1 ? i + j : i0;
#pragma unroll
        for (int tt = 0; tt < Q3_GATE_TOKENS; ++tt) acc[tt] += wv[j] * su[tt * bw + at];
      }
    }
  }
#pragma unroll
  for (int tt = 0; tt < Q3_GATE_TOKENS; ++tt) part[(quarter * 64 + lane) * Q3_GATE_TOKENS + tt] = acc[tt];
  __syncthreads();
  if (quarter == 0 && o < bw) {
    const float start = bias[((size_t)g * blocks + b) * bw + o];
#pragma unroll
    for (int tt = 0; tt < Q3_GATE_TOKENS; ++tt) {
      float total = start;
      for (int qtr = 0; qtr < 4; ++qtr) total += part[(qtr * 64 + lane) * Q3_GATE_TOKENS + tt];
      if (t0 + tt < T) out[((size_t)g * T + t0 + tt) * width + b * bw + o] = sigmoid_value(total);
    }
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
// One block per (sequence, head, 256 columns of the head's vdim), thread v keeps column v of S
// (dim x vdim) in registers. Rows of the input are [q: H dim | k: H dim | v: H vdim | g: H vdim]. Per
// token q and k turn by the position (pairs (i, i + half) of their first 2 * half numbers, angle =
// position * inv_freq[i]), k times k_scale; S = decay S + k v^T, o = S^T q, left as float32 in
// `raw` (T, H vdim): the division by the head's root mean square and the gate follow in
// retention_finish_kernel.
template <typename TA, int DMAX>
__global__ void __launch_bounds__(256) retention_scan_kernel(
    const TA* __restrict__ rows, const float* __restrict__ inv_freq, int half, const int* __restrict__ positions,
    const float* __restrict__ decays, float k_scale, float* __restrict__ state, long state_stride,
    const int* __restrict__ slots, const int* __restrict__ cu, float* __restrict__ raw, int H, int dim, int vdim) {
  __shared__ float sq[DMAX], sk[DMAX];
  const int slices = (vdim + 255) / 256;
  const int h = blockIdx.x / slices;
  const int v = (blockIdx.x % slices) * 256 + threadIdx.x;
  const int b = blockIdx.y;
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
    __syncthreads();
    for (int j = threadIdx.x; j < dim; j += 256) {
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
    if (live) raw[(size_t)t * hv + h * vdim + v] = acc;
  }
  if (live) {
#pragma unroll
    for (int n = 0; n < DMAX; ++n)
      if (n < dim) mine[(size_t)n * vdim] = S[n];
  }
}

// ---- recurrences with a decayed outer-product state, many tokens at a time ----
// Mamba-2 and retention are both   S_t = a_t S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t   per head, with
// a_t = exp(ld_t) <= 1 (retention: a constant per head; Mamba-2: exp(-rate step_t), q = C, k = B,
// v = step_t x_t). A sequence's rows are cut into chunks of 64. With la_t the sum of ld over the
// chunk's rows up to and including t, and S the state before the chunk:
//   o_t = exp(la_t) S^T q_t + sum_{s <= t} exp(la_t - la_s) (q_t . k_s) v_s
//   S'  = exp(la_last) S + sum_s exp(la_last - la_s) k_s v_s^T
// Three kernels: every chunk's own sum of outer products (all chunks at once); the states before
// every chunk, one chunk after the other (a multiply-add per number and chunk); every chunk's
// results (all chunks at once). Inputs are float32: q and k (T, groups, d), heads_per_group heads
// share a group's q and k; v (T, H, dv); ld[t * ld_row + h] (ld_row 0: one number per head).
#define Q3_CHUNK 64

__device__ inline int chunks_before(const int* __restrict__ cu, int b) {
  int n = 0;
  for (int i = 0; i < b; ++i) n += (cu[i + 1] - cu[i] + Q3_CHUNK - 1) / Q3_CHUNK;
  return n;
}

// la of the chunk's rows into shared memory (one thread; 64 additions), returns nothing.
__device__ inline void chunk_decays(float* la, const float* __restrict__ ld, long ld_row, int h, int row0, int len) {
  if (threadIdx.x == 0) {
    float run = 0.f;
    for (int s = 0; s < Q3_CHUNK; ++s) {
      if (s < len) run += ld[(size_t)(row0 + s) * ld_row + h];
      la[s] = run;
    }
  }
}

// grid (chunks of the longest sequence, H * dv tiles of 64, B); 256 threads. U[i][j] = sum_s
// exp(la_last - la_s) k_s[i] v_s[j] for the tile's 64 columns j, into `sums` (chunk, H, d, dv); the chunk's
// whole decay exp(la_last) into `decays` (chunk, H). All threads bring k and v into shared memory; then eight
// threads for every eight rows of d form 8 x 8 numbers each from 16-byte reads, four reads for 64 multiply-adds.
__global__ void __launch_bounds__(256) chunk_state_kernel(const float* __restrict__ k, const float* __restrict__ v,
                                                          const float* __restrict__ ld, long ld_row,
                                                          const int* __restrict__ cu, float* __restrict__ sums,
                                                          float* __restrict__ decays, int H, int hpg, int d, int dv) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int dp = (d + 7) / 8 * 8;           // rows of 8: the last ones may be zeros
  float* kw = lds;                          // (64, dp)
  float* vt = kw + Q3_CHUNK * dp;           // (64, 64)
  __shared__ float la[Q3_CHUNK];
  const int b = blockIdx.z;
  const int tiles = (dv + 63) / 64;
  const int h = blockIdx.y / tiles, tile = blockIdx.y % tiles;
  const int start = cu[b], n = cu[b + 1] - start;
  const int c = blockIdx.x;
  if (c * Q3_CHUNK >= n) return;
  const int row0 = start + c * Q3_CHUNK;
  const int len = n - c * Q3_CHUNK < Q3_CHUNK ? n - c * Q3_CHUNK : Q3_CHUNK;
  const int chunk = chunks_before(cu, b) + c;
  const int G = H / hpg, g = h / hpg;
  chunk_decays(la, ld, ld_row, h, row0, len);
  __syncthreads();
  const float last = la[len - 1];
  // sixteen loads a thread are asked for before the first is used (a loop of single loads is a chain of round trips)
  for (int e0 = threadIdx.x; e0 < Q3_CHUNK * dp; e0 += 256 * 16) {
    float got[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int e = e0 + 256 * u;
      const int s = e / dp, i = e % dp;
      got[u] = (e < Q3_CHUNK * dp && s < len && i < d) ? k[((size_t)(row0 + s) * G + g) * d + i] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int e = e0 + 256 * u;
      if (e < Q3_CHUNK * dp) kw[e] = e / dp < len ? got[u] * expf(last - la[e / dp]) : 0.f;
    }
  }
  {
    float got[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int e = threadIdx.x + 256 * u;
      const int s = e / 64, j = tile * 64 + e % 64;
      got[u] = (s < len && j < dv) ? v[((size_t)(row0 + s) * H + h) * dv + j] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) vt[threadIdx.x + 256 * u] = got[u];
  }
  __syncthreads();
  // (d up to 256: 32 groups of eight rows, eight threads each)
  const int ti = threadIdx.x / 8, tj = threadIdx.x % 8;      // rows 8 ti .., columns 8 tj ..
  if (8 * ti < dp) {
    float acc[8][8];
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
      for (int x = 0; x < 8; ++x) acc[r][x] = 0.f;
    for (int s = 0; s < len; ++s) {
      const float4 k0 = *reinterpret_cast<const float4*>(kw + s * dp + 8 * ti);
      const float4 k1 = *reinterpret_cast<const float4*>(kw + s * dp + 8 * ti + 4);
      const float4 v0 = *reinterpret_cast<const float4*>(vt + s * 64 + 8 * tj);
      const float4 v1 = *reinterpret_cast<const float4*>(vt + s * 64 + 8 * tj + 4);
      const float kk[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
      const float vv[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
      for (int r = 0; r < 8; ++r)
#pragma unroll
        for (int x = 0; x < 8; ++x) acc[r][x] += kk[r] * vv[x];
    }
    float* dst = sums + ((size_t)chunk * H + h) * d * dv;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int i = 8 * ti + r;
      if (i < d) {
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          const int j = tile * 64 + 8 * tj + x;
          if (j < dv) dst[(size_t)i * dv + j] = acc[r][x];
        }
      }
    }
  }
  if (tile == 0 && threadIdx.x == 0) decays[(size_t)chunk * H + h] = expf(last);
}

// grid (d * dv / 256, H, B): one number of the state per thread, through the sequence's chunks in
// order. `sums` receives, in place of each chunk's own sum, the state before that chunk; the state
// tensor receives the state after the last.
__global__ void chunk_scan_kernel(float* __restrict__ sums, const float* __restrict__ decays, float* __restrict__ state,
                                  long state_stride, const int* __restrict__ slots, const int* __restrict__ cu, int H,
                                  int size) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  if (e >= size) return;
  const int n = cu[b + 1] - cu[b];
  if (n <= 0) return;
  const int chunks = (n + Q3_CHUNK - 1) / Q3_CHUNK;
  const int first = chunks_before(cu, b);
  float* mine = state + (size_t)slots[b] * state_stride + (size_t)h * size + e;
  float S = *mine;
  for (int c = 0; c < chunks; ++c) {
    float* at = sums + ((size_t)(first + c) * H + h) * size + e;
    const float own = *at;
    *at = S;
    S = decays[(size_t)(first + c) * H + h] * S + own;
  }
  *mine = S;
}

// grid (chunks of the longest sequence, groups, B): the chunk's raw products q_t . k_s (64 x 64), over d in
// slices of 64 through shared memory, into `scores` (chunk, group, t, s). They are the same for all heads of a
// group and all tiles of a head's columns, which only weigh them with their own decays.
__global__ void __launch_bounds__(256) chunk_scores_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                           const int* __restrict__ cu, float* __restrict__ scores, int G,
                                                           int d) {
  __shared__ float one[Q3_CHUNK * 65];
  __shared__ float two[Q3_CHUNK * 65];
  const int b = blockIdx.z, g = blockIdx.y, c = blockIdx.x;
  const int start = cu[b], n = cu[b + 1] - start;
  if (c * Q3_CHUNK >= n) return;
  const int row0 = start + c * Q3_CHUNK;
  const int len = n - c * Q3_CHUNK < Q3_CHUNK ? n - c * Q3_CHUNK : Q3_CHUNK;
  const int chunk = chunks_before(cu, b) + c;
  const int tt = threadIdx.x / 16, tj = threadIdx.x % 16;
  float acc[4][4];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int x = 0; x < 4; ++x) acc[r][x] = 0.f;
  for (int i0 = 0; i0 < d; i0 += 64) {
    __syncthreads();
    {
      float gq[16], gk[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int e = threadIdx.x + 256 * u;
        const int s = e / 64, i = i0 + e % 64;
        const bool in = s < len && i < d;
        gq[u] = in ? q[((size_t)(row0 + s) * G + g) * d + i] : 0.f;
        gk[u] = in ? k[((size_t)(row0 + s) * G + g) * d + i] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int e = threadIdx.x + 256 * u;
        one[(e / 64) * 65 + e % 64] = gq[u];
        two[(e / 64) * 65 + e % 64] = gk[u];
      }
    }
    __syncthreads();
    for (int i = 0; i < 64; ++i) {
      float qv[4], kv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) qv[r] = one[(tt + 16 * r) * 65 + i];
#pragma unroll
      for (int x = 0; x < 4; ++x) kv[x] = two[(4 * tj + x) * 65 + i];
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int x = 0; x < 4; ++x) acc[r][x] += qv[r] * kv[x];
    }
  }
  float* dst = scores + ((size_t)chunk * G + g) * Q3_CHUNK * Q3_CHUNK;
#pragma unroll
  for (int r = 0; r < 4; ++r)
    *reinterpret_cast<float4*>(dst + (tt + 16 * r) * Q3_CHUNK + 4 * tj) = make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
}

// grid as chunk_state_kernel. A[t][s] = scores[t][s] exp(la_t - la_s) for s <= t; then
// o[t][j] = sum_s A[t][s] v_s[j] + exp(la_t) sum_i q_t[i] S[i][j] with S the state before the chunk (from `sums`),
// in slices of 64 over i through shared memory.
__global__ void __launch_bounds__(256) chunk_output_kernel(const float* __restrict__ q, const float* __restrict__ scores,
                                                           const float* __restrict__ v, const float* __restrict__ ld,
                                                           long ld_row, const int* __restrict__ cu,
                                                           const float* __restrict__ sums, float* __restrict__ out, int H,
                                                           int hpg, int d, int dv) {
  __shared__ float A[Q3_CHUNK * Q3_CHUNK];       // (t, s)
  __shared__ float one[Q3_CHUNK * 65];           // a slice of q, rows padded to 65
  __shared__ float two[Q3_CHUNK * 64];           // a slice of S, then of v
  __shared__ float la[Q3_CHUNK];
  const int b = blockIdx.z;
  const int tiles = (dv + 63) / 64;
  const int h = blockIdx.y / tiles, tile = blockIdx.y % tiles;
  const int start = cu[b], n = cu[b + 1] - start;
  const int c = blockIdx.x;
  if (c * Q3_CHUNK >= n) return;
  const int row0 = start + c * Q3_CHUNK;
  const int len = n - c * Q3_CHUNK < Q3_CHUNK ? n - c * Q3_CHUNK : Q3_CHUNK;
  const int chunk = chunks_before(cu, b) + c;
  const int G = H / hpg, g = h / hpg;
  chunk_decays(la, ld, ld_row, h, row0, len);
  __syncthreads();
  const int tt = threadIdx.x / 16, tj = threadIdx.x % 16;      // rows tt + 16 r, columns 4 tj .. 4 tj + 3
  float acc[4][4];
  const float* raw = scores + ((size_t)chunk * G + g) * Q3_CHUNK * Q3_CHUNK;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int t = tt + 16 * r;
    const float4 sc = *reinterpret_cast<const float4*>(raw + t * Q3_CHUNK + 4 * tj);
    const float got[4] = {sc.x, sc.y, sc.z, sc.w};
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int s = 4 * tj + x;
      A[t * Q3_CHUNK + s] = (s <= t && t < len) ? got[x] * expf(la[t] - la[s]) : 0.f;
      acc[r][x] = 0.f;
    }
  }
  // the state's share: exp(la_t) q_t S, a slice of 64 of d at a time
  const float* S = sums + ((size_t)chunk * H + h) * d * dv;
  for (int i0 = 0; i0 < d; i0 += 64) {
    __syncthreads();
    {
      float gq[16], gs[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int e = threadIdx.x + 256 * u;
        const int s = e / 64, i = i0 + e % 64;
        gq[u] = (s < len && i < d) ? q[((size_t)(row0 + s) * G + g) * d + i] : 0.f;
        const int si = i0 + e / 64, j = tile * 64 + e % 64;
        gs[u] = (si < d && j < dv) ? S[(size_t)si * dv + j] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int e = threadIdx.x + 256 * u;
        one[(e / 64) * 65 + e % 64] = gq[u];
        two[e] = gs[u];
      }
    }
    __syncthreads();
    for (int i = 0; i < 64; ++i) {
      const float4 sv = *reinterpret_cast<const float4*>(two + i * 64 + 4 * tj);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float qv = one[(tt + 16 * r) * 65 + i];
        acc[r][0] += qv * sv.x;
        acc[r][1] += qv * sv.y;
        acc[r][2] += qv * sv.z;
        acc[r][3] += qv * sv.w;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float grow = expf(la[tt + 16 * r]);
#pragma unroll
    for (int x = 0; x < 4; ++x) acc[r][x] *= grow;
  }
  // the chunk's own share: A v
  __syncthreads();
  {
    float gv[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int e = threadIdx.x + 256 * u;
      const int s = e / 64, j = tile * 64 + e % 64;
      gv[u] = (s < len && j < dv) ? v[((size_t)(row0 + s) * H + h) * dv + j] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) two[threadIdx.x + 256 * u] = gv[u];
  }
  __syncthreads();
  for (int s = 0; s < len; ++s) {
    const float4 vv = *reinterpret_cast<const float4*>(two + s * 64 + 4 * tj);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float a = A[(tt + 16 * r) * Q3_CHUNK + s];
      acc[r][0] += a * vv.x;
      acc[r][1] += a * vv.y;
      acc[r][2] += a * vv.z;
      acc[r][3] += a * vv.w;
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int t = tt + 16 * r;
    if (t < len) {
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int j = tile * 64 + 4 * tj + x;
        if (j < dv) out[((size_t)(row0 + t) * H + h) * dv + j] = acc[r][x];
      }
    }
  }
}

// What the three kernels need of Mamba-2's rows: step = softplus(dt + dt_bias); ld = -exp(A_log) step;
// v = step x; q = C, k = B as float32.
template <typename TA>
__global__ void mamba2_prepare_kernel(const TA* __restrict__ xbc, const TA* __restrict__ dt, long dt_stride,
                                      const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                      float* __restrict__ qf, float* __restrict__ kf, float* __restrict__ vf,
                                      float* __restrict__ ld, int H, int P, int N, int G) {
  extern __shared__ float step_of_head[];      // (H): a head's step is formed once, not once per column
  const int t = blockIdx.x;
  const int C = H * P + 2 * G * N;
  const TA* row = xbc + (size_t)t * C;
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    const float step = softplus_value(to_float(dt[(size_t)t * dt_stride + h]) + dt_bias[h]);
    step_of_head[h] = step;
    ld[(size_t)t * H + h] = -expf(a_log[h]) * step;
  }
  __syncthreads();
  for (int e0 = threadIdx.x; e0 < H * P; e0 += blockDim.x * 8) {
    float got[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int e = e0 + blockDim.x * u;
      got[u] = e < H * P ? to_float(row[e]) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int e = e0 + blockDim.x * u;
      if (e < H * P) vf[(size_t)t * H * P + e] = step_of_head[e / P] * got[u];
    }
  }
  for (int e = threadIdx.x; e < G * N; e += blockDim.x) {
    kf[(size_t)t * G * N + e] = to_float(row[H * P + e]);
    qf[(size_t)t * G * N + e] = to_float(row[H * P + G * N + e]);
  }
}

// y += D x after the three kernels.
template <typename TA>
__global__ void mamba2_skip_kernel(const TA* __restrict__ xbc, const float* __restrict__ d_skip, float* __restrict__ y,
                                   int H, int P, int C) {
  const int t = blockIdx.x;
  for (int e = threadIdx.x; e < H * P; e += blockDim.x)
    y[(size_t)t * H * P + e] += d_skip[e / P] * to_float(xbc[(size_t)t * C + e]);
}

// Retention's rows for the three kernels: q and k turned by the position (k times k_scale), v as float32.
template <typename TA>
__global__ void retention_prepare_kernel(const TA* __restrict__ rows, const float* __restrict__ inv_freq, int half,
                                         const int* __restrict__ positions, float k_scale, float* __restrict__ qf,
                                         float* __restrict__ kf, float* __restrict__ vf, int H, int dim, int vdim) {
  const int t = blockIdx.x;
  const int hd = H * dim, hv = H * vdim;
  const TA* row = rows + (size_t)t * (2 * (size_t)hd + 2 * (size_t)hv);
  const float pos = (float)positions[t];
  for (int e = threadIdx.x; e < hd; e += blockDim.x) {
    const int j = e % dim;
    float qv = to_float(row[e]), kv = to_float(row[hd + e]);
    if (j < 2 * half) {
      const bool first = j < half;
      const int partner = first ? e + half : e - half;
      const float angle = pos * inv_freq[first ? j : j - half];
      const float c = cosf(angle), s = sinf(angle);
      const float qp = to_float(row[partner]), kp = to_float(row[hd + partner]);
      qv = first ? qv * c - qp * s : qv * c + qp * s;
      kv = first ? kv * c - kp * s : kv * c + kp * s;
    }
    qf[(size_t)t * hd + e] = qv;
    kf[(size_t)t * hd + e] = kv * k_scale;
  }
  for (int e = threadIdx.x; e < hv; e += blockDim.x) vf[(size_t)t * hv + e] = to_float(row[2 * hd + e]);
}

// One block per (token, head): o divided by its root mean square over the head's vdim numbers, times silu(g).
template <typename TA>
__global__ void retention_finish_kernel(const float* __restrict__ o, const TA* __restrict__ rows, float eps,
                                        TA* __restrict__ out, int H, int dim, int vdim) {
  __shared__ float scratch[17];
  const int t = blockIdx.x, h = blockIdx.y;
  const int hd = H * dim, hv = H * vdim;
  const float* src = o + ((size_t)t * H + h) * vdim;
  const TA* gate = rows + (size_t)t * (2 * (size_t)hd + 2 * (size_t)hv) + 2 * hd + hv + h * vdim;
  float sq = 0.f;
  for (int j = threadIdx.x; j < vdim; j += blockDim.x) sq += src[j] * src[j];
  const float inv = rsqrtf(block_sum(sq, scratch) / (float)vdim + eps);
  for (int j = threadIdx.x; j < vdim; j += blockDim.x)
    out[(size_t)t * hv + h * vdim + j] = from_float<TA>(src[j] * inv * silu_value(to_float(gate[j])));
}

// Floats of workspace for a step of T rows in B sequences: q, k, v, ld, the chunks' sums, decays and raw scores.
extern "C" long q3_chunked_workspace(int T, int B, int H, int G, int d, int dv) {
  const long chunks = T / Q3_CHUNK + B;
  return 2L * T * G * d + (long)T * H * dv + (long)T * H + chunks * H * ((long)d * dv + 1) + chunks * G * Q3_CHUNK * Q3_CHUNK;
}

static int launch_chunks(const float* qf, const float* kf, const float* vf, const float* ld, long ld_row, float* sums,
                         float* decays, float* scores, float* state, long state_stride, const int* slots, const int* cu, float* out,
                         int B, int max_q_len, int H, int hpg, int d, int dv, hipStream_t stream) {
  const int chunks = (max_q_len + Q3_CHUNK - 1) / Q3_CHUNK;
  const int tiles = (dv + 63) / 64;
  const dim3 grid(chunks, H * tiles, B);
  const int dp = (d + 7) / 8 * 8;
  const size_t lds = (size_t)(Q3_CHUNK * dp + Q3_CHUNK * 64) * sizeof(float);
  if (lds > 64 * 1024) {
    // 64 rows of more than 192 numbers and the values' tile pass the 64 KB a launch may ask for unasked
    const hipError_t allowed = hipFuncSetAttribute(reinterpret_cast<const void*>(chunk_state_kernel),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (allowed != hipSuccess) return (int)allowed;
  }
  hipLaunchKernelGGL(chunk_state_kernel, grid, dim3(256), lds, stream, kf, vf, ld, ld_row, cu, sums, decays, H, hpg, d,
                     dv);
  hipLaunchKernelGGL(chunk_scan_kernel, dim3((d * dv + 255) / 256, H, B), dim3(256), 0, stream, sums, decays, state,
                     state_stride, slots, cu, H, d * dv);
  hipLaunchKernelGGL(chunk_scores_kernel, dim3(chunks, H / hpg, B), dim3(256), 0, stream, qf, kf, cu, scores, H / hpg, d);
  hipLaunchKernelGGL(chunk_output_kernel, grid, dim3(256), 0, stream, qf, scores, vf, ld, ld_row, cu, sums, out, H, hpg, d,
                     dv);
  return q3_launch_status();
}

extern "C" int q3_mamba2_chunked(const void* xbc, const void* dt, long dt_stride, const float* dt_bias,
                                 const float* a_log, const float* d_skip, float* state, long state_stride,
                                 const int* slots, const int* cu, float* y, float* workspace, int T, int B,
                                 int max_q_len, int H, int P, int N, int G, int act_dtype, hipStream_t stream) {
  if (T <= 0 || B <= 0 || H <= 0 || P <= 0 || N <= 0 || G <= 0 || H % G || max_q_len <= 0 || B > 65535)
    return Q3_ERR_BAD_ARGUMENT;
  if (N > 256 || (long)H * ((P + 63) / 64) > 65535) return Q3_ERR_UNSUPPORTED;
  float* scores = workspace;        // first: it is read and written sixteen bytes at a time
  float* qf = scores + (size_t)(T / Q3_CHUNK + B) * G * Q3_CHUNK * Q3_CHUNK;
  float* kf = qf + (size_t)T * G * N;
  float* vf = kf + (size_t)T * G * N;
  float* ld = vf + (size_t)T * H * P;
  float* sums = ld + (size_t)T * H;
  float* decays = sums + (size_t)(T / Q3_CHUNK + B) * H * N * P;
  Q3_DISPATCH_DTYPE(act_dtype, TA,
                    hipLaunchKernelGGL(mamba2_prepare_kernel<TA>, dim3(T), dim3(256), (size_t)H * sizeof(float), stream, (const TA*)xbc,
                                       (const TA*)dt, dt_stride, dt_bias, a_log, qf, kf, vf, ld, H, P, N, G));
  const int status = launch_chunks(qf, kf, vf, ld, H, sums, decays, scores, state, state_stride, slots, cu, y, B, max_q_len, H,
                                   H / G, N, P, stream);
  if (status) return status;
  Q3_DISPATCH_DTYPE(act_dtype, TA,
                    hipLaunchKernelGGL(mamba2_skip_kernel<TA>, dim3(T), dim3(256), 0, stream, (const TA*)xbc, d_skip, y,
                                       H, P, H * P + 2 * G * N));
  return q3_launch_status();
}

extern "C" int q3_retention_chunked(const void* rows, const float* inv_freq, int half, const int* positions,
                                    const float* log_decays, float k_scale, float eps, float* state, long state_stride,
                                    const int* slots, const int* cu, void* out, float* workspace, float* scratch_out,
                                    int T, int B, int max_q_len, int H, int dim, int vdim, int act_dtype,
                                    hipStream_t stream) {
  if (T <= 0 || B <= 0 || H <= 0 || dim <= 0 || vdim <= 0 || half < 0 || 2 * half > dim || max_q_len <= 0 || B > 65535 ||
      H > 65535)
    return Q3_ERR_BAD_ARGUMENT;
  if (half > 0 && !inv_freq) return Q3_ERR_BAD_ARGUMENT;
  if (dim > 256 || (long)H * ((vdim + 63) / 64) > 65535) return Q3_ERR_UNSUPPORTED;
  float* scores = workspace;
  float* qf = scores + (size_t)(T / Q3_CHUNK + B) * H * Q3_CHUNK * Q3_CHUNK;
  float* kf = qf + (size_t)T * H * dim;
  float* vf = kf + (size_t)T * H * dim;
  float* ld = vf + (size_t)T * H * vdim;          // unused stretch: the decays are one number per head
  float* sums = ld + (size_t)T * H;
  float* decays = sums + (size_t)(T / Q3_CHUNK + B) * H * dim * vdim;
  Q3_DISPATCH_DTYPE(act_dtype, TA,
                    hipLaunchKernelGGL(retention_prepare_kernel<TA>, dim3(T), dim3(256), 0, stream, (const TA*)rows,
                                       inv_freq, half, positions, k_scale, qf, kf, vf, H, dim, vdim));
  const int status = launch_chunks(qf, kf, vf, log_decays, 0, sums, decays, scores, state, state_stride, slots, cu, scratch_out,
                                   B, max_q_len, H, 1, dim, vdim, stream);
  if (status) return status;
  const int threads = vdim >= 256 ? 256 : (vdim >= 128 ? 128 : 64);
  Q3_DISPATCH_DTYPE(act_dtype, TA,
                    hipLaunchKernelGGL(retention_finish_kernel<TA>, dim3(T, H), dim3(threads), 0, stream, scratch_out,
                                       (const TA*)rows, eps, (TA*)out, H, dim, vdim));
  return q3_launch_status();
}

// The recurrent unit's recurrence over long sequences, in segments of 64 rows: every segment's own
// product of decays and its state from nothing (all segments at once), the states at the segments'
// starts one after the other, then every segment again from its true start.
__device__ inline void rglru_step(float& S, float k, float r, float i, float u) {
  const float log_a = -k * r;
  S = expf(log_a) * S + sqrtf(-expm1f(2.f * log_a)) * i * u;
}

__global__ void rglru_segment_kernel(const float* __restrict__ u, const float* __restrict__ gates,
                                     const float* __restrict__ rate, const int* __restrict__ cu, float* __restrict__ seg_decay,
                                     float* __restrict__ seg_state, int T, int width) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int b = blockIdx.z, seg = blockIdx.x;
  const int start = cu[b], n = cu[b + 1] - start;
  if (c >= width || seg * Q3_CHUNK >= n) return;
  const int first = start + seg * Q3_CHUNK;
  const int last = first + (n - seg * Q3_CHUNK < Q3_CHUNK ? n - seg * Q3_CHUNK : Q3_CHUNK);
  const float k = rate[c];
  float S = 0.f, logs = 0.f;
  for (int t = first; t < last; t += 8) {        // eight rows' inputs asked for at once
    float r[8], gi[8], uu[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const size_t at = (size_t)(t + j < last ? t + j : t) * width + c;
      r[j] = gates[at], gi[j] = gates[(size_t)T * width + at], uu[j] = u[at];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (t + j < last) {
        logs += -k * r[j];
        rglru_step(S, k, r[j], gi[j], uu[j]);
      }
    }
  }
  const size_t to = (size_t)(chunks_before(cu, b) + seg) * width + c;
  seg_decay[to] = expf(logs);
  seg_state[to] = S;
}

__global__ void rglru_carry_kernel(const float* __restrict__ seg_decay, float* __restrict__ seg_state,
                                   float* __restrict__ state, long state_stride, const int* __restrict__ slots,
                                   const int* __restrict__ cu, int width) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int b = blockIdx.y;
  const int n = cu[b + 1] - cu[b];
  if (c >= width || n <= 0) return;
  const int segments = (n + Q3_CHUNK - 1) / Q3_CHUNK, first = chunks_before(cu, b);
  float* mine = state + (size_t)slots[b] * state_stride + c;
  float S = *mine;
  for (int seg = 0; seg < segments; ++seg) {
    const size_t at = (size_t)(first + seg) * width + c;
    const float own = seg_state[at];
    seg_state[at] = S;
    S = seg_decay[at] * S + own;
  }
  *mine = S;
}

template <typename TO>
__global__ void rglru_apply_kernel(const float* __restrict__ u, const float* __restrict__ gates,
                                   const float* __restrict__ rate, const float* __restrict__ y, long y_stride,
                                   const float* __restrict__ y_bias, const int* __restrict__ cu,
                                   const float* __restrict__ seg_state, TO* __restrict__ out, int T, int width) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int b = blockIdx.z, seg = blockIdx.x;
  const int start = cu[b], n = cu[b + 1] - start;
  if (c >= width || seg * Q3_CHUNK >= n) return;
  const int first = start + seg * Q3_CHUNK;
  const int last = first + (n - seg * Q3_CHUNK < Q3_CHUNK ? n - seg * Q3_CHUNK : Q3_CHUNK);
  const float k = rate[c], yb = y_bias[c];
  float S = seg_state[(size_t)(chunks_before(cu, b) + seg) * width + c];
  for (int t = first; t < last; t += 8) {
    float r[8], gi[8], uu[8], yy[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = t + j < last ? t + j : t;
      const size_t at = (size_t)row * width + c;
      r[j] = gates[at], gi[j] = gates[(size_t)T * width + at], uu[j] = u[at], yy[j] = y[(size_t)row * y_stride + c];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (t + j < last) {
        rglru_step(S, k, r[j], gi[j], uu[j]);
        const float z = yy[j] + yb;
        out[(size_t)(t + j) * width + c] =
            from_float<TO>(S * (0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)))));
      }
    }
  }
}

// workspace: 2 * (T / 64 + B) * width floats
extern "C" int q3_rglru_chunked(const float* u, const float* gates, const float* rate, const float* y, long y_stride,
                                const float* y_bias, float* state, long state_stride, const int* slots, const int* cu,
                                void* out, float* workspace, int T, int B, int max_q_len, int width, int out_dtype,
                                hipStream_t stream) {
  if (T <= 0 || B <= 0 || width <= 0 || max_q_len <= 0 || B > 65535) return Q3_ERR_BAD_ARGUMENT;
  const int threads = width >= 256 ? 256 : 64;
  const int cols = (width + threads - 1) / threads;
  if (cols > 65535) return Q3_ERR_UNSUPPORTED;
  const dim3 grid((max_q_len + Q3_CHUNK - 1) / Q3_CHUNK, cols, B);
  float* seg_decay = workspace;
  float* seg_state = workspace + (size_t)(T / Q3_CHUNK + B) * width;
  hipLaunchKernelGGL(rglru_segment_kernel, grid, dim3(threads), 0, stream, u, gates, rate, cu, seg_decay, seg_state, T,
                     width);
  hipLaunchKernelGGL(rglru_carry_kernel, dim3(cols, B), dim3(threads), 0, stream, seg_decay, seg_state, state,
                     state_stride, slots, cu, width);
  Q3_DISPATCH_DTYPE(out_dtype, TO,
                    hipLaunchKernelGGL(rglru_apply_kernel<TO>, grid, dim3(threads), 0, stream, u, gates, rate, y, y_stride,
                                       y_bias, cu, seg_state, (TO*)out, T, width));
  return q3_launch_status();
}

// ---- launchers ----

extern "C" int q3_causal_conv(const void* x, long x_stride, const float* in_bias, const float* w, const float* bias,
                              float* state, long state_stride, const int* slots, const int* cu, const int* seq_index,
                              void* out, int T, int B, int C, int taps, int act, int single_rows, int in_dtype,
                              int out_dtype, hipStream_t stream) {
  if (T <= 0 || B <= 0 || C <= 0 || taps < 1 || taps > Q3_TAPS_MOST || act < 0 || act > 1) return Q3_ERR_BAD_ARGUMENT;
  const int threads = C >= 256 ? 256 : 64;
  const int chunks = (C + threads - 1) / threads;
  if (chunks > 65535) return Q3_ERR_UNSUPPORTED;
  // `single_rows`: every sequence brings exactly one row (T == B); the tail then moves in the same kernel
  const bool fused = single_rows && T == B && taps > 1;
  const int rows_each = fused ? 1 : (T >= 2048 ? 16 : (T >= 256 ? 4 : 1));
  const size_t in_size = in_dtype == Q3_F32 ? 4 : 2, out_size = out_dtype == Q3_F32 ? 4 : 2;
  if (!fused && T >= 256 && C % 8 == 0 && x_stride % 8 == 0 && ((size_t)x % 16) == 0 && ((size_t)out % 16) == 0 &&
      (x_stride * in_size) % 16 == 0 && (C * out_size) % 16 == 0 && ((size_t)bias % 16) == 0 && ((size_t)w % 16) == 0 &&
      (!in_bias || ((size_t)in_bias % 16) == 0)) {
    const int wide_threads = 64;       // the kernel's shared memory is sized for this
    const int wide_rows = Q3_CONV_TILE;
    Q3_DISPATCH_DTYPE(in_dtype, TI, Q3_DISPATCH_DTYPE(out_dtype, TO, {
                        hipLaunchKernelGGL((causal_conv_wide_kernel<TI, TO>),
                                           dim3((T + wide_rows - 1) / wide_rows, (C / 8 + wide_threads - 1) / wide_threads),
                                           dim3(wide_threads), 0, stream, (const TI*)x, x_stride, in_bias, w, bias, state,
                                           state_stride, slots, cu, seq_index, (TO*)out, T, C, taps, act, wide_rows);
                      }));
  } else
  Q3_DISPATCH_DTYPE(in_dtype, TI, Q3_DISPATCH_DTYPE(out_dtype, TO, {
                      hipLaunchKernelGGL((causal_conv_kernel<TI, TO>), dim3((T + rows_each - 1) / rows_each, chunks),
                                         dim3(threads), 0, stream, (const TI*)x, x_stride, in_bias, w, bias, state,
                                         state_stride, slots, cu, seq_index, (TO*)out, T, C, taps, act, rows_each,
                                         fused ? state : (float*)nullptr);
                    }));
  if (taps > 1 && !fused)
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
  if (T <= 96) {
    const int out_tiles = (bw + 63) / 64;
    if ((long)blocks * out_tiles > 65535) return Q3_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(block_gates_few_kernel, dim3((T + Q3_GATE_TOKENS - 1) / Q3_GATE_TOKENS, blocks * out_tiles, 2),
                       dim3(256), (size_t)(Q3_GATE_TOKENS * bw + 4 * 64 * Q3_GATE_TOKENS) * sizeof(float), stream, u, w,
                       bias, out, T, width, bw, out_tiles);
    return q3_launch_status();
  }
  const int out_tiles = (bw + 63) / 64;
  if ((long)blocks * out_tiles > 65535) return Q3_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(block_gates_kernel, dim3((T + 63) / 64, blocks * out_tiles, 2), dim3(256), 0, stream, u, w, bias, out,
                     T, width, bw, out_tiles);
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
                            void* out, float* raw, int T, int B, int H, int dim, int vdim, hipStream_t stream) {
  const dim3 grid(H * ((vdim + 255) / 256), B);
#define Q3_RETENTION(DMAX)                                                                                            \
  hipLaunchKernelGGL((retention_scan_kernel<TA, DMAX>), grid, dim3(256), 0, stream, (const TA*)rows, inv_freq, half,  \
                     positions, decays, k_scale, state, state_stride, slots, cu, raw, H, dim, vdim)
  if (dim <= 32) Q3_RETENTION(32);
  else if (dim <= 64) Q3_RETENTION(64);
  else if (dim <= 128) Q3_RETENTION(128);
  else Q3_RETENTION(256);
#undef Q3_RETENTION
  const int threads = vdim >= 256 ? 256 : (vdim >= 128 ? 128 : 64);
  hipLaunchKernelGGL(retention_finish_kernel<TA>, dim3(T, H), dim3(threads), 0, stream, raw, (const TA*)rows, eps,
                     (TA*)out, H, dim, vdim);
  return q3_launch_status();
}

// `raw`: float32 (T, H vdim) of scratch for the results before their norm and gate.
extern "C" int q3_retention_scan(const void* rows, const float* inv_freq, int half, const int* positions,
                                 const float* decays, float k_scale, float eps, float* state, long state_stride,
                                 const int* slots, const int* cu, void* out, float* raw, int T, int B, int H, int dim,
                                 int vdim, int act_dtype, hipStream_t stream) {
  if (T <= 0 || B <= 0 || H <= 0 || dim <= 0 || vdim <= 0 || half < 0 || 2 * half > dim || B > 65535 || !raw)
    return Q3_ERR_BAD_ARGUMENT;
  if (half > 0 && !inv_freq) return Q3_ERR_BAD_ARGUMENT;
  if (dim > 256 || (long)H * ((vdim + 255) / 256) > 65535) return Q3_ERR_UNSUPPORTED;
  Q3_DISPATCH_DTYPE(act_dtype, TA, return launch_retention<TA>(rows, inv_freq, half, positions, decays, k_scale, eps,
                                                               state, state_stride, slots, cu, out, raw, T, B, H, dim,
                                                               vdim, stream));
  return 0;
}
