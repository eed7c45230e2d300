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
// One block per token. `down` (T, q_rank + kv_rank + rot_dim) is the joint down-projection.
//   cq[t]    = rms_norm(down[t, :q_rank]) * q_weight                       -> (T, q_rank)
//   cache row of (sequence, position) = [rms_norm(down[t, q_rank:q_rank+kv_rank]) * kv_weight |
//                                        rotate(down[t, q_rank+kv_rank:])]
// The rotation turns pairs (2i, 2i+1), i < rot_pairs, by angle = float(position) * inv_freq[i]
// (a float32 product), with cos and sin multiplied by rot_factor; numbers beyond 2 rot_pairs pass.
// ---------------------------------------------------------------------------
template <typename T, typename W>
__global__ void latent_prepare_kernel(const T* __restrict__ down, int q_rank, int kv_rank, int rot_dim,
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
  const T* src = down + (size_t)t * R;
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
// y[t, h, :] = W[h]^T x[t, h, :] for every head: x rows of `I` numbers at x + t * x_row + h * x_head,
// W (H, I, O) row-major (the summed index first), y rows of `O` numbers at out + t * out_row +
// h * out_head. One block: 16 tokens of one head, up to 256 output columns; the tokens' inputs
// wait in shared memory, each thread owns one output column and walks I in order.
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
  const T* wh = w + (size_t)h * I * O + o;
  for (int i = 0; i < I; ++i) {
    const float wv = to_float(wh[(size_t)i * O]);
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] += xs[m * I + i] * wv;
  }
  for (int m = 0; m < rows; ++m)
    out[(size_t)(m0 + m) * out_row + (size_t)h * out_head + o] = from_float<T>(acc[m]);
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
// positions j <= p, and with a window w > 0 only p - j < w.
// ---------------------------------------------------------------------------
#define LAT_BM 16
#define LAT_BN 32

template <typename T, int NV>
__global__ __launch_bounds__(256) void latent_attn_kernel(const T* __restrict__ q, T* __restrict__ out,
                                                          const T* __restrict__ cache, int num_pages,
                                                          const int* __restrict__ block_table, int bt_stride,
                                                          const int* __restrict__ cu_q,
                                                          const int* __restrict__ kv_lens, int H, int Dk, int Dv,
                                                          int page, float scale, int window) {
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
    const float inv = 1.f / l_run;
    T* o = out + ((size_t)(q0 + my_tok) * H + my_head) * Dv;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int col = sub + 16 * i;
      if (col < Dv) o[col] = from_float<T>(acc[i] * inv);
    }
  }
}

static int raise_shared_memory(const void* kernel, size_t smem) {
  if (smem <= 48 * 1024) return 0;
  if (smem > 160 * 1024) return Q3_ERR_UNSUPPORTED;
  return (int)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
}

extern "C" int q3_latent_prepare(const void* down, int T, int q_rank, int kv_rank, int rot_dim, const void* q_weight,
                                 const void* kv_weight, int w_dtype, float eps, const float* inv_freq, int rot_pairs,
                                 float rot_factor, const int* positions, const int* seq_index,
                                 const int* block_table, int bt_stride, int bt_rows, void* cache, int page,
                                 int num_pages, void* cq, int dtype, hipStream_t stream) {
  if (T <= 0 || q_rank <= 0 || kv_rank <= 0 || rot_dim <= 0 || 2 * rot_pairs > rot_dim || rot_pairs < 0)
    return Q3_ERR_BAD_ARGUMENT;
  if (cache && (!block_table || page <= 0 || num_pages <= 0 || bt_stride <= 0)) return Q3_ERR_BAD_ARGUMENT;
  const int R = q_rank + kv_rank + rot_dim;
  const size_t smem = (size_t)(32 + R) * sizeof(float);
  int threads = 64;
  while (threads < 512 && threads * 2 < R) threads *= 2;
  Q3_DISPATCH_DTYPE(dtype, TT, Q3_DISPATCH_DTYPE(w_dtype, WW, {
    int e = raise_shared_memory((const void*)latent_prepare_kernel<TT, WW>, smem);
    if (e) return e;
    hipLaunchKernelGGL((latent_prepare_kernel<TT, WW>), dim3(T), dim3(threads), smem, stream, (const TT*)down, q_rank,
                       kv_rank, rot_dim, (const WW*)q_weight, (const WW*)kv_weight, eps, inv_freq, rot_pairs,
                       rot_factor, positions, seq_index, block_table, bt_stride, bt_rows, (TT*)cache, page, num_pages,
                       (TT*)cq);
    return q3_launch_status();
  }));
  return Q3_ERR_BAD_ARGUMENT;
}

extern "C" int q3_headwise_linear(const void* x, long x_row, int x_head, const void* w, void* out, long out_row,
                                  int out_head, int n_rows, int H, int I, int O, int dtype, hipStream_t stream) {
  if (n_rows <= 0 || H <= 0 || I <= 0 || O <= 0 || H > 65535) return Q3_ERR_BAD_ARGUMENT;
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
                              int page, float scale, int window, int max_q_len, hipStream_t stream) {
  const size_t smem = (size_t)(LAT_BM * Dk + LAT_BN * (Dk + 1) + LAT_BM * (LAT_BN + 1)) * sizeof(float);
  int e = raise_shared_memory((const void*)latent_attn_kernel<T, NV>, smem);
  if (e) return e;
  const long tiles = ((long)max_q_len * H + LAT_BM - 1) / LAT_BM;
  if (tiles > 0x7fffffffL || B > 65535) return Q3_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((latent_attn_kernel<T, NV>), dim3((unsigned)tiles, B), dim3(256), smem, stream, (const T*)q,
                     (T*)out, (const T*)cache, num_pages, block_table, bt_stride, cu_q, kv_lens, H, Dk, Dv, page, scale,
                     window);
  return q3_launch_status();
}

extern "C" int q3_latent_attention(const void* q, void* out, const void* cache, int num_pages, const int* block_table,
                                   int bt_stride, const int* cu_q, const int* kv_lens, int B, int H, int Dk, int Dv,
                                   int page, float scale, int window, int max_q_len, int dtype, hipStream_t stream) {
  if (B <= 0 || H <= 0 || Dk <= 0 || Dv <= 0 || Dv > Dk || page <= 0 || max_q_len <= 0 || window < 0)
    return Q3_ERR_BAD_ARGUMENT;
  if (Dv > 1024) return Q3_ERR_UNSUPPORTED;
  Q3_DISPATCH_DTYPE(dtype, TT, {
    if (Dv <= 128)
      return launch_latent_attn<TT, 8>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, H, Dk, Dv,
                                       page, scale, window, max_q_len, stream);
    if (Dv <= 256)
      return launch_latent_attn<TT, 16>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, H, Dk, Dv,
                                        page, scale, window, max_q_len, stream);
    if (Dv <= 512)
      return launch_latent_attn<TT, 32>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, H, Dk, Dv,
                                        page, scale, window, max_q_len, stream);
    return launch_latent_attn<TT, 64>(q, out, cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B, H, Dk, Dv,
                                      page, scale, window, max_q_len, stream);
  });
  return Q3_ERR_BAD_ARGUMENT;
}
