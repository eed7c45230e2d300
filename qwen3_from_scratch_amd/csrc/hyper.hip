// A residual held in several streams (hyper-connections): the embedding into equal streams, the
// kernel that lets a sublayer's result into all streams, reads them for the next sublayer and
// applies a layer norm, all in float32; a gated root-mean-square norm in equal parts; a weighted
// sum of two tensors.
#include "common.h"

#define Q3_STREAMS_MOST 8

// out[t, s, :] = float(table[ids[t], :]) for every stream s.
template <typename T>
__global__ void embed_streams_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                     float* __restrict__ out, int S, int W, int V) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;
  const T* row = table + (size_t)(ok ? id : 0) * W;
  float* dst = out + (size_t)t * S * W;
  for (int j = threadIdx.x; j < W; j += blockDim.x) {
    const float v = ok ? to_float(row[j]) : 0.f;
    for (int s = 0; s < S; ++s) dst[(size_t)s * W + j] = v;
  }
}

// One block per output row r (source row src = rows[r], or r). With `delta`:
//   x_t <- sum_s mix[s, t] x_s + write[t] * delta        (all t from the old streams; written back if asked)
// then u = sum_s read[s] x_s (read null: the plain sum), and with `weight`
//   out = (u - mean u) * rsqrt(mean (u - mean u)^2 + eps) * weight,
// the mean taken first and the deviations squared afterwards. u stays in shared memory between
// the passes. Everything is float32; `out` is rounded once.
template <typename TA, int VEC>
__global__ void hyper_norm_kernel(float* __restrict__ x, const TA* __restrict__ delta, const float* __restrict__ mix,
                                  const float* __restrict__ write, const float* __restrict__ read,
                                  const float* __restrict__ weight, const int* __restrict__ rows,
                                  TA* __restrict__ out, int S, int W, float eps, int write_back) {
  extern __shared__ float u_row[];
  __shared__ float scratch[17];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  // the tables are the same for every thread: scalar loads, no staging and no barrier before the streams' loads
  float s_mix[Q3_STREAMS_MOST * Q3_STREAMS_MOST], s_write[Q3_STREAMS_MOST], s_read[Q3_STREAMS_MOST];
#pragma unroll
  for (int i = 0; i < Q3_STREAMS_MOST; ++i) {
    s_write[i] = (write && i < S) ? write[i] : 0.f;
    s_read[i] = i < S ? (read ? read[i] : 1.f) : 0.f;
#pragma unroll
    for (int t = 0; t < Q3_STREAMS_MOST; ++t) s_mix[i * Q3_STREAMS_MOST + t] = (mix && i < S && t < S) ? mix[i * S + t] : 0.f;
  }
  float* xs = x + src * S * W;
  float sum = 0.f;
  // VEC columns a thread and turn (four where the width allows: 16-byte loads and stores of the streams)
  for (int j = threadIdx.x * VEC; j < W; j += blockDim.x * VEC) {
    float old[Q3_STREAMS_MOST][VEC];
#pragma unroll
    for (int s = 0; s < Q3_STREAMS_MOST; ++s) {
      if (s < S) {
        if constexpr (VEC == 4) {
          const float4 v = *reinterpret_cast<const float4*>(xs + (size_t)s * W + j);
          old[s][0] = v.x, old[s][1] = v.y, old[s][2] = v.z, old[s][3] = v.w;
        } else {
          old[s][0] = xs[(size_t)s * W + j];
        }
      }
    }
    float u[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) u[e] = 0.f;
    if (delta) {
      float d[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) d[e] = to_float(delta[src * W + j + e]);
#pragma unroll
      for (int t = 0; t < Q3_STREAMS_MOST; ++t) {
        if (t < S) {
          float v[VEC];
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            v[e] = 0.f;
#pragma unroll
            for (int s = 0; s < Q3_STREAMS_MOST; ++s)
              if (s < S) v[e] += s_mix[s * Q3_STREAMS_MOST + t] * old[s][e];
            v[e] += s_write[t] * d[e];
            u[e] += s_read[t] * v[e];
          }
          if (write_back) {
            if constexpr (VEC == 4)
              *reinterpret_cast<float4*>(xs + (size_t)t * W + j) = make_float4(v[0], v[1], v[2], v[3]);
            else
              xs[(size_t)t * W + j] = v[0];
          }
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < Q3_STREAMS_MOST; ++s)
        if (s < S) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) u[e] += s_read[s] * old[s][e];
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      u_row[j + e] = u[e];
      sum += u[e];
    }
  }
  if (!out) return;
  const float mean = block_sum(sum, scratch) / (float)W;
  float sq = 0.f;
  for (int j = threadIdx.x; j < W; j += blockDim.x) {
    const float d = u_row[j] - mean;
    sq += d * d;
  }
  const float inv = rsqrtf(block_sum(sq, scratch) / (float)W + eps);
  TA* dst = out + (size_t)r * W;
  for (int j = threadIdx.x; j < W; j += blockDim.x) dst[j] = from_float<TA>((u_row[j] - mean) * inv * weight[j]);
}

// One block per (token, part): v = y * silu(gate); out = v * rsqrt(mean(v^2) + eps) * weight over
// the part's `size` numbers. y float32 (T, inner); gate rows `gate_stride` apart.
template <typename TA>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ y, const TA* __restrict__ gate, long gate_stride,
                                     const float* __restrict__ weight, TA* __restrict__ out, int inner, int size,
                                     float eps) {
  __shared__ float scratch[17];
  const int t = blockIdx.x, part = blockIdx.y;
  const float* yr = y + (size_t)t * inner + (size_t)part * size;
  const TA* gr = gate + (size_t)t * gate_stride + (size_t)part * size;
  float sq = 0.f;
  for (int j = threadIdx.x; j < size; j += blockDim.x) {
    const float g = to_float(gr[j]);
    const float v = yr[j] * (g / (1.f + expf(-g)));
    sq += v * v;
  }
  const float inv = rsqrtf(block_sum(sq, scratch) / (float)size + eps);
  TA* dst = out + (size_t)t * inner + (size_t)part * size;
  const float* w = weight + (size_t)part * size;
  for (int j = threadIdx.x; j < size; j += blockDim.x) {
    const float g = to_float(gr[j]);
    dst[j] = from_float<TA>(yr[j] * (g / (1.f + expf(-g))) * inv * w[j]);
  }
}

template <typename TA>
__global__ void scaled_sum_kernel(const TA* __restrict__ a, float alpha, const TA* __restrict__ b, float beta,
                                  TA* __restrict__ out, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    out[i] = from_float<TA>(alpha * to_float(a[i]) + beta * to_float(b[i]));
}

static inline int threads_for(int n) { return n >= 1024 ? 256 : (n >= 256 ? 128 : 64); }

extern "C" int q3_embed_streams(const int* ids, const void* table, float* out, int T, int S, int W, int V,
                                int table_dtype, hipStream_t stream) {
  if (T <= 0 || S <= 0 || W <= 0 || V <= 0) return Q3_ERR_BAD_ARGUMENT;
  Q3_DISPATCH_DTYPE(table_dtype, TT,
                    hipLaunchKernelGGL(embed_streams_kernel<TT>, dim3(T), dim3(threads_for(W)), 0, stream, ids,
                                       (const TT*)table, out, S, W, V));
  return q3_launch_status();
}

extern "C" int q3_hyper_norm(float* x, const void* delta, const float* mix, const float* write, const float* read,
                             const float* weight, const int* rows, void* out, int n_out, int S, int W, float eps,
                             int act_dtype, int write_back, hipStream_t stream) {
  if (n_out <= 0 || S <= 0 || S > Q3_STREAMS_MOST || W <= 0) return Q3_ERR_BAD_ARGUMENT;
  if ((size_t)W * sizeof(float) > 60 * 1024) return Q3_ERR_UNSUPPORTED;
  if (delta && (!mix || !write)) return Q3_ERR_BAD_ARGUMENT;
  if (out && !weight) return Q3_ERR_BAD_ARGUMENT;
  if (W % 4 == 0)
    Q3_DISPATCH_DTYPE(act_dtype, TA,
                      hipLaunchKernelGGL((hyper_norm_kernel<TA, 4>), dim3(n_out), dim3(W >= 2048 ? 512 : threads_for(W / 2)),
                                         (size_t)W * sizeof(float), stream, x, (const TA*)delta, mix, write, read, weight,
                                         rows, (TA*)out, S, W, eps, write_back));
  else
    Q3_DISPATCH_DTYPE(act_dtype, TA,
                      hipLaunchKernelGGL((hyper_norm_kernel<TA, 1>), dim3(n_out), dim3(threads_for(W)),
                                         (size_t)W * sizeof(float), stream, x, (const TA*)delta, mix, write, read, weight,
                                         rows, (TA*)out, S, W, eps, write_back));
  return q3_launch_status();
}

extern "C" int q3_gated_rmsnorm(const float* y, const void* gate, long gate_stride, const float* weight, void* out,
                                int T, int inner, int parts, float eps, int act_dtype, hipStream_t stream) {
  if (T <= 0 || inner <= 0 || parts <= 0 || inner % parts || parts > 65535) return Q3_ERR_BAD_ARGUMENT;
  const int size = inner / parts;
  Q3_DISPATCH_DTYPE(act_dtype, TA,
                    hipLaunchKernelGGL(gated_rmsnorm_kernel<TA>, dim3(T, parts), dim3(threads_for(size)), 0, stream, y,
                                       (const TA*)gate, gate_stride, weight, (TA*)out, inner, size, eps));
  return q3_launch_status();
}

extern "C" int q3_scaled_sum(const void* a, float alpha, const void* b, float beta, void* out, long n, int dtype,
                             hipStream_t stream) {
  if (n <= 0) return Q3_ERR_BAD_ARGUMENT;
  long blocks = (n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  Q3_DISPATCH_DTYPE(dtype, TA, hipLaunchKernelGGL(scaled_sum_kernel<TA>, dim3((unsigned)blocks), dim3(256), 0, stream,
                                                  (const TA*)a, alpha, (const TA*)b, beta, (TA*)out, (size_t)n));
  return q3_launch_status();
}
