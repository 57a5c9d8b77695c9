// Kernels of decoders with a 32-bit residual stream, latent (low-rank, shared-key) attention and
// group-limited sigmoid routing, for gfx950.  Every kernel exists for bf16 and for fp32 activations
// (dtype 0 / 1 in the entry points); what a design computes in 32-bit (norms, angles, scores,
// softmax, routing, the residual sum) is fp32 in both.
//
//   embed_scale        residual[t] = embed[id[t]] * scale                                (fp32 out)
//   add_rmsnorm        residual += delta;  y = residual * rsqrt(mean(residual^2) + eps) * w
//   rmsnorm_rows       y = x * rsqrt(mean(x^2) + eps) * w over a column range of a wider row
//   latent_kv_write    a token's compressed KV entry: RMS-normed latent | rotated shared key part
//                      -> paged cache row [rank + rot]
//   rope_pairs         interleaved-pair rotary embedding of a column range of every head, in place
//   latent_attention   causal attention of query rows in latent space over the paged entries with an
//                      optional per-head sink logit in the softmax denominator
//   sigmoid_gate       y[t, h, :] *= sigmoid(g[t, h])
//   relu_sq            y = relu(x)^2
//   glu_clamp          y = g' * sigmoid(alpha g') * (u' + bias),  g' = min(g, limit), u' = clamp(u, +-limit)
//   group_topk         sigmoid scores -> best groups by the sum of their two largest -> top-k experts
//   route_softmax      softmax scores (+ a selection bias) -> best groups by their largest biased score -> top-k;
//                      trailing identity experts leave the pair list and come back as one gate per token
//   rmsnorm_add        residual += rmsnorm(delta) * w;  y = residual (activation dtype)
//   gated_add_rmsnorm  residual += sigmoid(gate + b) (.) (c1 n1(d1) + c2 n2(d2)) + extra + vector;  y = rmsnorm(residual) w
//   glu_act            silu(g) * u  or  gelu_tanh(g) * u  of  x = g | u
//   gather_rows        xs[r] = x[idx[r]]
//   moe_finish         residual[t] += sum_k w[t,k] * y[pos[t,k]] + gate[t] * shared[t]
//
// Sizes are free (no multiple-of-8 requirements): these are the plain kernels every shape can take.
#include "common.h"

namespace {

template <typename T> struct Conv;
template <> struct Conv<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Conv<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return (float)*p; }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = (bf16_t)v; }
};

__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_reduce_sum(v);
  const int tid = threadIdx.x;
  __syncthreads();
  if ((tid & 63) == 0) red[tid >> 6] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) s += red[i];
  return s;
}

__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_reduce_max(v);
  const int tid = threadIdx.x;
  __syncthreads();
  if ((tid & 63) == 0) red[tid >> 6] = v;
  __syncthreads();
  float s = red[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) s = fmaxf(s, red[i]);
  return s;
}

__device__ __forceinline__ float sigmoidf(float x) { return 1.f / (1.f + expf(-x)); }

// ---------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void embed_scale_kernel(const long* __restrict__ ids, const T* __restrict__ embed,
                                                          float* __restrict__ out, int width, float scale) {
  const long row = blockIdx.x;
  const T* e = embed + ids[row] * (long)width;
  float* o = out + row * width;
  for (int i = threadIdx.x; i < width; i += 256) o[i] = Conv<T>::ld(e + i) * scale;
}

// residual fp32 [rows, n] (+= delta, row stride d_stride) -> y (row stride y_stride)
template <typename T>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                                          long d_stride, const float* __restrict__ w,
                                                          T* __restrict__ y, long y_stride, int n, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* r = residual + row * n;
  float ss = 0.f;
  if (delta) {
    const T* d = delta + row * d_stride;
    for (int i = threadIdx.x; i < n; i += 256) {
      const float v = r[i] + Conv<T>::ld(d + i);
      r[i] = v;  // read back below by the same thread
      ss += v * v;
    }
  } else {
    for (int i = threadIdx.x; i < n; i += 256) {
      const float v = r[i];
      ss += v * v;
    }
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
  if (!y) return;
  T* yr = y + row * y_stride;
  for (int i = threadIdx.x; i < n; i += 256) Conv<T>::st(yr + i, r[i] * inv * w[i]);
}

template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const T* __restrict__ x, long x_stride,
                                                           const float* __restrict__ w, T* __restrict__ y,
                                                           long y_stride, int n, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const T* xr = x + row * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = Conv<T>::ld(xr + i);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
  T* yr = y + row * y_stride;
  for (int i = threadIdx.x; i < n; i += 256) Conv<T>::st(yr + i, Conv<T>::ld(xr + i) * inv * w[i]);
}

// x [rows, >= rank + rot] (row stride x_stride): columns [0, rank) are RMS-normed with w, columns
// [rank, rank + rot) are the shared key part, whose first rot_dims columns rotate in interleaved
// pairs (2i, 2i+1) by the angle table cos_sin[pos] = cos[0 .. rot_dims/2) | sin[0 .. rot_dims/2).
// The entry goes to cache + (slot / 64) * page_stride + (slot % 64) * (rank + rot); slot < 0 skips.
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(const T* __restrict__ x, long x_stride,
                                                              const float* __restrict__ w,
                                                              const int* __restrict__ positions,
                                                              const long* __restrict__ slots,
                                                              const float* __restrict__ cos_sin, T* __restrict__ cache,
                                                              long page_stride, int rank, int rot, int rot_dims,
                                                              float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const long slot = slots[row];
  if (slot < 0) return;
  const T* xr = x + row * x_stride;
  T* dst = cache + (slot / PAGE) * page_stride + (slot % PAGE) * (long)(rank + rot);
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += 256) {
    const float v = Conv<T>::ld(xr + i);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += 256) Conv<T>::st(dst + i, Conv<T>::ld(xr + i) * inv * w[i]);
  const int half = rot_dims >> 1;
  const float* cs = cos_sin + (long)positions[row] * rot_dims;
  for (int i = threadIdx.x; i < half; i += 256) {
    const float u = Conv<T>::ld(xr + rank + 2 * i), v = Conv<T>::ld(xr + rank + 2 * i + 1);
    const float c = cs[i], s = cs[half + i];
    Conv<T>::st(dst + rank + 2 * i, u * c - v * s);
    Conv<T>::st(dst + rank + 2 * i + 1, v * c + u * s);
  }
  for (int i = rot_dims + threadIdx.x; i < rot; i += 256) dst[rank + i] = xr[rank + i];
}

// q [rows, heads, head_stride]: columns [col0, col0 + rot_dims) of every head rotate in place
template <typename T>
__global__ __launch_bounds__(256) void rope_pairs_kernel(T* __restrict__ q, long row_stride, long head_stride,
                                                         const int* __restrict__ positions,
                                                         const float* __restrict__ cos_sin, int heads, int col0,
                                                         int rot_dims) {
  const long row = blockIdx.x;
  const int half = rot_dims >> 1;
  const float* cs = cos_sin + (long)positions[row] * rot_dims;
  for (int i = threadIdx.x; i < heads * half; i += 256) {
    const int h = i / half, j = i % half;
    T* p = q + row * row_stride + h * head_stride + col0 + 2 * j;
    const float u = Conv<T>::ld(p), v = Conv<T>::ld(p + 1);
    const float c = cs[j], s = cs[half + j];
    Conv<T>::st(p, u * c - v * s);
    Conv<T>::st(p + 1, v * c + u * s);
  }
}

// ---------------------------------------------------------------------------------
// Latent attention, plain form.  One 256-thread workgroup per (query row, head).  The query is
// q_lat [rank] (the head's unrotated query carried into latent space) | q_rot [rot]; key j of the
// row's sequence is the cache entry [rank + rot] and its value the entry's first rank columns.
//   score_j = (q_lat . c_j + q_rot . r_j) * scale,   j <= position
//   out     = sum_j exp(score_j - m) c_j / (sum_j exp(score_j - m) + exp(sink - m))
// Keys are taken 256 at a time (a thread scores one key, then owns output columns tid, tid+256, ..).
// ---------------------------------------------------------------------------------
#define LAT_MAX_COLS 8  // rank <= 2048

template <typename T>
__global__ __launch_bounds__(256) void latent_attention_kernel(
    const T* __restrict__ q_lat, long ql_row, long ql_head, const T* __restrict__ q_rot, long qr_row, long qr_head,
    const T* __restrict__ cache, long page_stride, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ row_seq, const int* __restrict__ positions, const float* __restrict__ sink,
    T* __restrict__ out, long o_row, long o_head, int rank, int rot, float scale) {
  extern __shared__ float smem[];
  float* qs = smem;             // [rank + rot], pre-scaled
  float* ps = smem + rank + rot;  // [256]
  __shared__ float red[4];
  const int row = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int width = rank + rot;
  const int ctx = positions[row] + 1;
  const int seq = row_seq ? row_seq[row] : row;
  const int* bt = block_tables + (long)seq * bt_stride;
  for (int i = tid; i < rank; i += 256) qs[i] = Conv<T>::ld(q_lat + row * ql_row + h * ql_head + i) * scale;
  for (int i = tid; i < rot; i += 256) qs[rank + i] = Conv<T>::ld(q_rot + row * qr_row + h * qr_head + i) * scale;
  float m = sink ? sink[h] : -INFINITY;
  float l = sink ? 1.f : 0.f;
  float acc[LAT_MAX_COLS];
#pragma unroll
  for (int c = 0; c < LAT_MAX_COLS; ++c) acc[c] = 0.f;
  __syncthreads();
  for (int j0 = 0; j0 < ctx; j0 += 256) {
    const int j = j0 + tid;
    float s = -INFINITY;
    if (j < ctx) {
      const T* k = cache + (long)bt[j / PAGE] * page_stride + (long)(j % PAGE) * width;
      float a = 0.f;
      for (int d = 0; d < width; ++d) a += qs[d] * Conv<T>::ld(k + d);
      s = a;
    }
    const float mc = block_max(s, red);
    const float mn = fmaxf(m, mc);
    const float p = j < ctx ? expf(s - mn) : 0.f;
    const float corr = (m == -INFINITY) ? 0.f : expf(m - mn);
    ps[tid] = p;
    const float psum = block_sum(p, red);  // (its barriers also publish ps)
    l = l * corr + psum;
    m = mn;
    const int nk = min(256, ctx - j0);
#pragma unroll
    for (int c = 0; c < LAT_MAX_COLS; ++c) {
      const int d = c * 256 + tid;
      if (d < rank) {
        float a = acc[c] * corr;
        for (int jj = 0; jj < nk; ++jj) {
          const int key = j0 + jj;
          a += ps[jj] * Conv<T>::ld(cache + (long)bt[key / PAGE] * page_stride + (long)(key % PAGE) * width + d);
        }
        acc[c] = a;
      }
    }
    __syncthreads();  // ps is rewritten by the next 256 keys
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int c = 0; c < LAT_MAX_COLS; ++c) {
    const int d = c * 256 + tid;
    if (d < rank) Conv<T>::st(out + row * o_row + h * o_head + d, acc[c] * inv);
  }
}

// y [rows, heads, vdim] (contiguous) *= sigmoid(g[row * g_stride + head])
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(T* __restrict__ y, const T* __restrict__ g, long g_stride,
                                                           int heads, int vdim) {
  const long row = blockIdx.x;
  T* yr = y + row * heads * vdim;
  for (int i = threadIdx.x; i < heads * vdim; i += 256) {
    const float s = sigmoidf(Conv<T>::ld(g + row * g_stride + i / vdim));
    Conv<T>::st(yr + i, Conv<T>::ld(yr + i) * s);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void relu_sq_kernel(const T* __restrict__ x, T* __restrict__ y, long n) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const float v = fmaxf(Conv<T>::ld(x + i), 0.f);
    Conv<T>::st(y + i, v * v);
  }
}

// x [rows, 2 * inter] (row stride x_stride): gate columns then up columns -> y [rows, inter]
template <typename T>
__global__ __launch_bounds__(256) void glu_clamp_kernel(const T* __restrict__ x, long x_stride, T* __restrict__ y,
                                                        int inter, long total, float limit, float alpha,
                                                        float up_bias) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const long r = i / inter;
    const int c = (int)(i % inter);
    const float g = fminf(Conv<T>::ld(x + r * x_stride + c), limit);
    const float u = fminf(fmaxf(Conv<T>::ld(x + r * x_stride + inter + c), -limit), limit);
    Conv<T>::st(y + i, g * sigmoidf(alpha * g) * (u + up_bias));
  }
}

// ---------------------------------------------------------------------------------
// Group-limited top-k routing on sigmoid scores.  logits fp32 [tokens, cols] (cols >= experts; with
// `extra` column `experts` holds a per-token gate logit whose sigmoid goes to extra_out).  Experts
// form `groups` equal runs of neighbours; a group scores the sum of its two largest scores (its
// only one for groups of one); experts outside the `keep` best groups cannot be chosen.  Weights
// are the chosen scores times route_scale (not renormalised).  Ties go to the lower index.
// One wave per token.
// ---------------------------------------------------------------------------------
#define ROUTE_MAX_EXPERTS 1024

__global__ __launch_bounds__(64) void group_topk_kernel(const float* __restrict__ logits, int cols,
                                                        float* __restrict__ weights, int* __restrict__ ids,
                                                        float* __restrict__ extra_out, int experts, int groups,
                                                        int keep, int topk, float route_scale, int normalize) {
  // normalize: the chosen scores are divided by their sum (+ 1e-20) before route_scale
  __shared__ float s[ROUTE_MAX_EXPERTS];
  __shared__ float gs[ROUTE_MAX_EXPERTS];
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = logits + t * cols;
  for (int e = lane; e < experts; e += 64) s[e] = sigmoidf(z[e]);
  if (extra_out && lane == 0) extra_out[t] = sigmoidf(z[experts]);
  __syncthreads();
  const int per = experts / groups;
  for (int g = lane; g < groups; g += 64) {
    float a = -1.f, b = -1.f;  // two largest (scores are > 0)
    for (int e = g * per; e < (g + 1) * per; ++e) {
      const float v = s[e];
      if (v > a) { b = a; a = v; }
      else if (v > b) { b = v; }
    }
    gs[g] = per > 1 ? a + b : a;
  }
  __syncthreads();
  // the keep best groups: group g stays when fewer than keep groups beat it (a tie counts for the lower index)
  for (int g = lane; g < groups; g += 64) {
    int ahead = 0;
    const float v = gs[g];
    for (int o = 0; o < groups; ++o) ahead += (gs[o] > v) || (gs[o] == v && o < g);
    if (ahead >= keep)
      for (int e = g * per; e < (g + 1) * per; ++e) s[e] = -1.f;
  }
  __syncthreads();
  for (int k = 0; k < topk; ++k) {
    float best = -2.f;
    int bi = 0x7fffffff;
    for (int e = lane; e < experts; e += 64)
      if (s[e] > best) { best = s[e]; bi = e; }
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (lane == 0) {
      weights[t * topk + k] = best * route_scale;
      ids[t * topk + k] = bi;
    }
    __syncthreads();
    if (lane == 0) s[bi] = -3.f;
    __syncthreads();
  }
  if (normalize && lane == 0) {
    float sum = 0.f;
    for (int k = 0; k < topk; ++k) sum += weights[t * topk + k];
    const float inv = 1.f / (sum / route_scale + 1e-20f);
    for (int k = 0; k < topk; ++k) weights[t * topk + k] *= inv;
  }
}

// Softmax routing with a selection bias.  Scores s = softmax(z) over all n outputs; an expert is chosen by
// c = s + bias, weighted by s.  Experts form `groups` equal runs of neighbours, a group scores its largest c and
// only the `keep` best groups take part (the rest count as minus infinity; c may be negative).  The last
// n - experts outputs are identity experts: a chosen one adds its score to gate[t] and leaves the pair list
// (weight 0, id = park).  Ties go to the lower index.  One wave per token.
__global__ __launch_bounds__(64) void route_softmax_kernel(const float* __restrict__ logits, int cols,
                                                           const float* __restrict__ bias,
                                                           float* __restrict__ weights, int* __restrict__ ids,
                                                           float* __restrict__ gate, int n, int experts, int groups,
                                                           int keep, int topk, float route_scale, int park) {
  __shared__ float s[ROUTE_MAX_EXPERTS];
  __shared__ float c[ROUTE_MAX_EXPERTS];
  __shared__ float gs[ROUTE_MAX_EXPERTS];
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = logits + t * cols;
  float mx = -INFINITY;
  for (int e = lane; e < n; e += 64) mx = fmaxf(mx, z[e]);
  mx = wave_reduce_max(mx);
  float sum = 0.f;
  for (int e = lane; e < n; e += 64) {
    const float v = expf(z[e] - mx);
    s[e] = v;
    sum += v;
  }
  sum = wave_reduce_sum(sum);
  __syncthreads();
  for (int e = lane; e < n; e += 64) {
    const float v = s[e] / sum;
    s[e] = v;
    c[e] = v + (bias ? bias[e] : 0.f);
  }
  __syncthreads();
  const int per = n / groups;
  for (int g = lane; g < groups; g += 64) {
    float a = -INFINITY;
    for (int e = g * per; e < (g + 1) * per; ++e) a = fmaxf(a, c[e]);
    gs[g] = a;
  }
  __syncthreads();
  for (int g = lane; g < groups; g += 64) {
    int ahead = 0;
    const float v = gs[g];
    for (int o = 0; o < groups; ++o) ahead += (gs[o] > v) || (gs[o] == v && o < g);
    if (ahead >= keep)
      for (int e = g * per; e < (g + 1) * per; ++e) c[e] = -INFINITY;
  }
  __syncthreads();
  float gsum = 0.f;
  for (int k = 0; k < topk; ++k) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < n; e += 64)
      if (c[e] > best) { best = c[e]; bi = e; }
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    const bool none = bi == 0x7fffffff;  // fewer candidates than topk: an empty pair
    if (lane == 0) {
      const bool ident = !none && bi >= experts;
      const float w = none ? 0.f : s[bi] * route_scale;
      if (ident) gsum += w;
      weights[t * topk + k] = (ident || none) ? 0.f : w;
      ids[t * topk + k] = (ident || none) ? park : bi;
    }
    __syncthreads();
    if (lane == 0 && !none) c[bi] = -INFINITY;
    __syncthreads();
  }
  if (lane == 0 && gate) gate[t] = gsum;
}

// residual fp32 [rows, n] += rmsnorm(delta) * w (a norm on a sublayer's OUTPUT); y = the new residual, rounded
template <typename T, typename D>
__global__ __launch_bounds__(256) void rmsnorm_add_kernel(float* __restrict__ residual, const D* __restrict__ delta,
                                                          long d_stride, const float* __restrict__ w,
                                                          T* __restrict__ y, int n, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* r = residual + row * n;
  const D* d = delta + row * d_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = Conv<D>::ld(d + i);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = r[i] + Conv<D>::ld(d + i) * inv * w[i];
    r[i] = v;
    if (y) Conv<T>::st(y + row * n + i, v);
  }
}

// A gated residual in front of a pre-norm.  Per row:
//   residual += sigmoid(gate + gate_bias) (.) (c1 n1(d1) + c2 n2(d2)) + extra + extra_vec;  y = rmsnorm(residual) w
// with n_i(d) = rmsnorm(d) w_i where a weight w_i is given and d itself otherwise.  Every part is optional: no gate
// means a plain add, no deltas only the extras (a second stream that re-enters, a vector per pass of a layer loop).
// d1 in D (the activation dtype, or fp32 for a mixture's sum), d2, gate and y in T.
__device__ __forceinline__ void ld8(const float* p, float* v) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = a[e], v[4 + e] = b[e];
}
__device__ __forceinline__ void ld8(const bf16_t* p, float* v) {
  const u32x4 a = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
  for (int e = 0; e < 4; ++e) v[2 * e] = bf16lo(a[e]), v[2 * e + 1] = bf16hi(a[e]);
}
__device__ __forceinline__ void st8(float* p, const float* v) {
  *reinterpret_cast<f32x4*>(p) = (f32x4){v[0], v[1], v[2], v[3]};
  *reinterpret_cast<f32x4*>(p + 4) = (f32x4){v[4], v[5], v[6], v[7]};
}
__device__ __forceinline__ void st8(bf16_t* p, const float* v) {
  *reinterpret_cast<u32x4*>(p) = (u32x4){pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]),
                                         pack_bf16x2(v[6], v[7])};
}

// K > 0: rows of up to 2048 K values, a multiple of 8, every operand on 16-byte boundaries: a thread owns runs of 8
// neighbouring values, loads every operand once with 16-byte loads and keeps the new stream in registers.
// K = 0: any width and alignment, value by value, operands read again where needed.
template <typename T, typename D, int K>
__global__ __launch_bounds__(256) void gated_add_rmsnorm_kernel(
    float* __restrict__ residual, const D* __restrict__ d1, long s1, const float* __restrict__ w1, float c1,
    const T* __restrict__ d2, long s2, const float* __restrict__ w2, float c2, const T* __restrict__ gate, long sg,
    const float* __restrict__ gate_bias, const float* __restrict__ extra, const float* __restrict__ extra_vec,
    const float* __restrict__ w, T* __restrict__ y, int n, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* r = residual + row * n;
  if constexpr (K > 0) {
    float a1[K][8], a2[K][8], x[K][8];
    float q1 = 0.f, q2 = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i = (threadIdx.x + 256 * k) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) a1[k][e] = a2[k][e] = 0.f;
      if (i < n) {
        if (d1) ld8(d1 + row * s1 + i, a1[k]);
        if (d2) ld8(d2 + row * s2 + i, a2[k]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) q1 += a1[k][e] * a1[k][e], q2 += a2[k][e] * a2[k][e];
    }
    float f1 = c1, f2 = c2;
    if (d1 && w1) f1 = c1 / sqrtf(block_sum(q1, red) / (float)n + eps);
    if (d2 && w2) f2 = c2 / sqrtf(block_sum(q2, red) / (float)n + eps);
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i = (threadIdx.x + 256 * k) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) x[k][e] = 0.f;
      if (i < n) {
        float t[8], u[8];
        ld8(r + i, x[k]);
        if (d1 && w1) {
          ld8(w1 + i, t);
#pragma unroll
          for (int e = 0; e < 8; ++e) a1[k][e] *= t[e];
        }
        if (d2 && w2) {
          ld8(w2 + i, t);
#pragma unroll
          for (int e = 0; e < 8; ++e) a2[k][e] *= t[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] = a1[k][e] * f1 + a2[k][e] * f2;
        if (gate) {
          ld8(gate + row * sg + i, u);
          if (gate_bias) {
            float b[8];
            ld8(gate_bias + i, b);
#pragma unroll
            for (int e = 0; e < 8; ++e) u[e] += b[e];
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) t[e] *= sigmoidf(u[e]);
        }
        if (extra) {
          ld8(extra + row * n + i, u);
#pragma unroll
          for (int e = 0; e < 8; ++e) t[e] += u[e];
        }
        if (extra_vec) {
          ld8(extra_vec + i, u);
#pragma unroll
          for (int e = 0; e < 8; ++e) t[e] += u[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) x[k][e] += t[e];
        if (d1 || d2 || extra || extra_vec) st8(r + i, x[k]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[k][e] * x[k][e];
    }
    if (!y) return;
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i = (threadIdx.x + 256 * k) * 8;
      if (i < n) {
        float t[8];
        ld8(w + i, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] *= x[k][e] * inv;
        st8(y + row * n + i, t);
      }
    }
  } else {
    float q1 = 0.f, q2 = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) {
      const float u = d1 ? Conv<D>::ld(d1 + row * s1 + i) : 0.f, v = d2 ? Conv<T>::ld(d2 + row * s2 + i) : 0.f;
      q1 += u * u;
      q2 += v * v;
    }
    float f1 = c1, f2 = c2;
    if (d1 && w1) f1 = c1 / sqrtf(block_sum(q1, red) / (float)n + eps);
    if (d2 && w2) f2 = c2 / sqrtf(block_sum(q2, red) / (float)n + eps);
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) {
      float d = 0.f;
      if (d1) d += Conv<D>::ld(d1 + row * s1 + i) * f1 * (w1 ? w1[i] : 1.f);
      if (d2) d += Conv<T>::ld(d2 + row * s2 + i) * f2 * (w2 ? w2[i] : 1.f);
      if (gate) d *= sigmoidf(Conv<T>::ld(gate + row * sg + i) + (gate_bias ? gate_bias[i] : 0.f));
      float v = r[i] + d;
      if (extra) v += extra[row * n + i];
      if (extra_vec) v += extra_vec[i];
      r[i] = v;  // read back below by the same thread
      ss += v * v;
    }
    if (!y) return;
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += 256) Conv<T>::st(y + row * n + i, r[i] * inv * w[i]);
  }
}

// x [rows, 2 inter] = gate | up  ->  act(gate) * up;  kind 0: silu, 1: gelu in its tanh form
template <typename T>
__global__ __launch_bounds__(256) void glu_act_kernel(const T* __restrict__ x, long x_stride, T* __restrict__ y,
                                                      int inter, long total, int kind) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const long row = i / inter;
    const int col = (int)(i - row * inter);
    const float g = Conv<T>::ld(x + row * x_stride + col);
    const float u = Conv<T>::ld(x + row * x_stride + inter + col);
    float a;
    if (kind == 0) a = g * sigmoidf(g);
    else a = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    Conv<T>::st(y + i, a * u);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gather_rows_kernel(const T* __restrict__ x, const int* __restrict__ idx,
                                                          T* __restrict__ xs, int n) {
  const long row = blockIdx.x;
  const T* src = x + (long)idx[row] * n;
  for (int i = threadIdx.x; i < n; i += 256) xs[row * n + i] = src[i];
}

template <typename T>
__global__ __launch_bounds__(256) void moe_finish_kernel(float* __restrict__ residual, const T* __restrict__ y,
                                                         const float* __restrict__ weights,
                                                         const int* __restrict__ pos, int topk,
                                                         const T* __restrict__ shared, const float* __restrict__ gate,
                                                         int n, int overwrite) {
  // overwrite: the sum replaces what `residual` held (a buffer of its own instead of a stream)
  const long t = blockIdx.x;
  const float sg = shared ? (gate ? gate[t] : 1.f) : 0.f;
  // the first pairs' weights and rows are read once, ahead of the walk over the channels (a launch of a few
  // tokens is bound by the chain weight -> row index -> value, not by bytes)
  constexpr int AHEAD = 8;
  float wk[AHEAD];
  const T* yk[AHEAD];
#pragma unroll
  for (int k = 0; k < AHEAD; ++k) {
    wk[k] = k < topk ? weights[t * topk + k] : 0.f;
    yk[k] = y + (long)(wk[k] != 0.f ? pos[t * topk + k] : 0) * n;
  }
  for (int i = threadIdx.x; i < n; i += 256) {
    float a = 0.f;
#pragma unroll
    for (int k = 0; k < AHEAD; ++k)
      if (wk[k] != 0.f) a += wk[k] * Conv<T>::ld(yk[k] + i);
    for (int k = AHEAD; k < topk; ++k) {
      const float w = weights[t * topk + k];
      if (w != 0.f) a += w * Conv<T>::ld(y + (long)pos[t * topk + k] * n + i);
    }
    if (shared) a += sg * Conv<T>::ld(shared + t * n + i);
    residual[t * n + i] = overwrite ? a : residual[t * n + i] + a;
  }
}

inline int flat_grid(long total) {
  long b = (total + 255) / 256;
  return (int)(b < 1 ? 1 : (b > 65535 ? 65535 : b));
}

}  // namespace

#define DISPATCH(dtype, CALL_BF16, CALL_F32) \
  do {                                       \
    if ((dtype) == 0) { CALL_BF16; }         \
    else if ((dtype) == 1) { CALL_F32; }     \
    else return -2;                          \
  } while (0)

VPSA_EXPORT int vpsa_embed_scale(const long* ids, const void* embed, float* out, int rows, int width, float scale,
                                 int dtype, hipStream_t st) {
  if (rows <= 0) return 0;
  DISPATCH(dtype,
           hipLaunchKernelGGL(embed_scale_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, ids, (const bf16_t*)embed, out, width, scale),
           hipLaunchKernelGGL(embed_scale_kernel<float>, dim3(rows), dim3(256), 0, st, ids, (const float*)embed, out, width, scale));
  return 0;
}

VPSA_EXPORT int vpsa_add_rmsnorm(float* residual, const void* delta, long d_stride, const float* w, void* y,
                                 long y_stride, int rows, int n, float eps, int dtype, hipStream_t st) {
  if (rows <= 0) return 0;
  DISPATCH(dtype,
           hipLaunchKernelGGL(add_rmsnorm_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, residual, (const bf16_t*)delta, d_stride, w, (bf16_t*)y, y_stride, n, eps),
           hipLaunchKernelGGL(add_rmsnorm_kernel<float>, dim3(rows), dim3(256), 0, st, residual, (const float*)delta, d_stride, w, (float*)y, y_stride, n, eps));
  return 0;
}

VPSA_EXPORT int vpsa_rmsnorm_rows(const void* x, long x_stride, const float* w, void* y, long y_stride, int rows,
                                  int n, float eps, int dtype, hipStream_t st) {
  if (rows <= 0) return 0;
  DISPATCH(dtype,
           hipLaunchKernelGGL(rmsnorm_rows_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (const bf16_t*)x, x_stride, w, (bf16_t*)y, y_stride, n, eps),
           hipLaunchKernelGGL(rmsnorm_rows_kernel<float>, dim3(rows), dim3(256), 0, st, (const float*)x, x_stride, w, (float*)y, y_stride, n, eps));
  return 0;
}

VPSA_EXPORT int vpsa_latent_kv_write(const void* x, long x_stride, const float* w, const int* positions,
                                     const long* slots, const float* cos_sin, void* cache, long page_stride,
                                     int rows, int rank, int rot, int rot_dims, float eps, int dtype,
                                     hipStream_t st) {
  if (rows <= 0) return 0;
  if (rot_dims > rot || (rot_dims & 1)) return -1;
  DISPATCH(dtype,
           hipLaunchKernelGGL(latent_kv_write_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (const bf16_t*)x, x_stride, w, positions, slots, cos_sin, (bf16_t*)cache, page_stride, rank, rot, rot_dims, eps),
           hipLaunchKernelGGL(latent_kv_write_kernel<float>, dim3(rows), dim3(256), 0, st, (const float*)x, x_stride, w, positions, slots, cos_sin, (float*)cache, page_stride, rank, rot, rot_dims, eps));
  return 0;
}

VPSA_EXPORT int vpsa_rope_pairs(void* q, long row_stride, long head_stride, const int* positions,
                                const float* cos_sin, int rows, int heads, int col0, int rot_dims, int dtype,
                                hipStream_t st) {
  if (rows <= 0 || rot_dims == 0) return 0;
  if (rot_dims & 1) return -1;
  DISPATCH(dtype,
           hipLaunchKernelGGL(rope_pairs_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (bf16_t*)q, row_stride, head_stride, positions, cos_sin, heads, col0, rot_dims),
           hipLaunchKernelGGL(rope_pairs_kernel<float>, dim3(rows), dim3(256), 0, st, (float*)q, row_stride, head_stride, positions, cos_sin, heads, col0, rot_dims));
  return 0;
}

VPSA_EXPORT int vpsa_latent_attention(const void* q_lat, long ql_row, long ql_head, const void* q_rot, long qr_row,
                                      long qr_head, const void* cache, long page_stride, const int* block_tables,
                                      int bt_stride, const int* row_seq, const int* positions, const float* sink,
                                      void* out, long o_row, long o_head, int rows, int heads, int rank, int rot,
                                      float scale, int dtype, hipStream_t st) {
  if (rows <= 0) return 0;
  if (rank > LAT_MAX_COLS * 256 || heads > 65535) return -1;
  const size_t lds = (size_t)(rank + rot + 256) * sizeof(float);
  if (lds > 60 * 1024) return -1;
  dim3 grid(rows, heads);
  DISPATCH(dtype,
           hipLaunchKernelGGL(latent_attention_kernel<bf16_t>, grid, dim3(256), lds, st, (const bf16_t*)q_lat, ql_row, ql_head, (const bf16_t*)q_rot, qr_row, qr_head, (const bf16_t*)cache, page_stride, block_tables, bt_stride, row_seq, positions, sink, (bf16_t*)out, o_row, o_head, rank, rot, scale),
           hipLaunchKernelGGL(latent_attention_kernel<float>, grid, dim3(256), lds, st, (const float*)q_lat, ql_row, ql_head, (const float*)q_rot, qr_row, qr_head, (const float*)cache, page_stride, block_tables, bt_stride, row_seq, positions, sink, (float*)out, o_row, o_head, rank, rot, scale));
  return 0;
}

VPSA_EXPORT int vpsa_sigmoid_gate(void* y, const void* g, long g_stride, int rows, int heads, int vdim, int dtype,
                                  hipStream_t st) {
  if (rows <= 0) return 0;
  DISPATCH(dtype,
           hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (bf16_t*)y, (const bf16_t*)g, g_stride, heads, vdim),
           hipLaunchKernelGGL(sigmoid_gate_kernel<float>, dim3(rows), dim3(256), 0, st, (float*)y, (const float*)g, g_stride, heads, vdim));
  return 0;
}

VPSA_EXPORT int vpsa_relu_sq(const void* x, void* y, long n, int dtype, hipStream_t st) {
  if (n <= 0) return 0;
  DISPATCH(dtype,
           hipLaunchKernelGGL(relu_sq_kernel<bf16_t>, dim3(flat_grid(n)), dim3(256), 0, st, (const bf16_t*)x, (bf16_t*)y, n),
           hipLaunchKernelGGL(relu_sq_kernel<float>, dim3(flat_grid(n)), dim3(256), 0, st, (const float*)x, (float*)y, n));
  return 0;
}

VPSA_EXPORT int vpsa_glu_clamp(const void* x, long x_stride, void* y, int rows, int inter, float limit, float alpha,
                               float up_bias, int dtype, hipStream_t st) {
  const long total = (long)rows * inter;
  if (total <= 0) return 0;
  DISPATCH(dtype,
           hipLaunchKernelGGL(glu_clamp_kernel<bf16_t>, dim3(flat_grid(total)), dim3(256), 0, st, (const bf16_t*)x, x_stride, (bf16_t*)y, inter, total, limit, alpha, up_bias),
           hipLaunchKernelGGL(glu_clamp_kernel<float>, dim3(flat_grid(total)), dim3(256), 0, st, (const float*)x, x_stride, (float*)y, inter, total, limit, alpha, up_bias));
  return 0;
}

VPSA_EXPORT int vpsa_group_topk(const float* logits, int cols, float* weights, int* ids, float* extra_out,
                                int tokens, int experts, int groups, int keep, int topk, float route_scale,
                                int normalize, hipStream_t st) {
  if (tokens <= 0) return 0;
  if (experts > ROUTE_MAX_EXPERTS || groups < 1 || experts % groups || keep < 1 || keep > groups ||
      topk > experts / groups * keep || cols < experts + (extra_out ? 1 : 0))
    return -1;
  hipLaunchKernelGGL(group_topk_kernel, dim3(tokens), dim3(64), 0, st, logits, cols, weights, ids, extra_out,
                     experts, groups, keep, topk, route_scale, normalize);
  return 0;
}

// d1_f32: the first delta is fp32 whatever the activation dtype (a mixture's fp32 sum)
VPSA_EXPORT int vpsa_gated_add_rmsnorm(float* residual, const void* d1, long s1, int d1_f32, const float* w1, float c1,
                                       const void* d2, long s2, const float* w2, float c2, const void* gate, long sg,
                                       const float* gate_bias, const float* extra, const float* extra_vec,
                                       const float* w, void* y, int rows, int n, float eps, int dtype, hipStream_t st) {
  if (rows <= 0) return 0;
  if (dtype != 0 && dtype != 1) return -2;
  if (y && !w) return -1;
#define GA_P(T, D, P)                                                                                                   \
  gated_add_rmsnorm_kernel<T, D, P><<<rows, 256, 0, st>>>(residual, (const D*)d1, s1, w1, c1, (const T*)d2, s2, w2, c2, \
                                                          (const T*)gate, sg, gate_bias, extra, extra_vec, w, (T*)y, n, eps)
  // 16-byte loads need every operand's rows on 16-byte boundaries
  auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  const bool vec = n % 8 == 0 && s1 % 8 == 0 && s2 % 8 == 0 && sg % 8 == 0 && al(residual) && al(d1) && al(w1) && al(d2) &&
                   al(w2) && al(gate) && al(gate_bias) && al(extra) && al(extra_vec) && al(w) && al(y);
#define GA(T, D)                                 \
  if (vec && n <= 2048) GA_P(T, D, 1);           \
  else if (vec && n <= 4096) GA_P(T, D, 2);      \
  else if (vec && n <= 8192) GA_P(T, D, 4);      \
  else GA_P(T, D, 0)
  if (dtype == 1) { GA(float, float); }
  else if (d1_f32) { GA(bf16_t, float); }
  else { GA(bf16_t, bf16_t); }
#undef GA
#undef GA_P
  return 0;
}

// park: the id a chosen identity expert's pair gets (its weight is 0): the expert count for callers that sort pairs
// into a bucket no product visits, 0 for callers that run every pair.
VPSA_EXPORT int vpsa_route_softmax(const float* logits, int cols, const float* bias, float* weights, int* ids,
                                   float* gate, int tokens, int n, int experts, int groups, int keep, int topk,
                                   float route_scale, int park, hipStream_t st) {
  if (tokens <= 0) return 0;
  if (n > ROUTE_MAX_EXPERTS || experts > n || groups < 1 || n % groups || keep < 1 || keep > groups || cols < n ||
      topk < 1 || (experts < n && !gate))
    return -1;
  hipLaunchKernelGGL(route_softmax_kernel, dim3(tokens), dim3(64), 0, st, logits, cols, bias, weights, ids, gate, n,
                     experts, groups, keep, topk, route_scale, park);
  return 0;
}

// delta_f32: the delta is fp32 whatever the activation dtype (a mixture's fp32 sum)
VPSA_EXPORT int vpsa_rmsnorm_add(float* residual, const void* delta, long d_stride, int delta_f32, const float* w,
                                 void* y, int rows, int n, float eps, int dtype, hipStream_t st) {
  if (rows <= 0) return 0;
  if (dtype != 0 && dtype != 1) return -2;
  if (dtype == 1)
    rmsnorm_add_kernel<float, float><<<rows, 256, 0, st>>>(residual, (const float*)delta, d_stride, w, (float*)y, n, eps);
  else if (delta_f32)
    rmsnorm_add_kernel<bf16_t, float><<<rows, 256, 0, st>>>(residual, (const float*)delta, d_stride, w, (bf16_t*)y, n, eps);
  else
    rmsnorm_add_kernel<bf16_t, bf16_t><<<rows, 256, 0, st>>>(residual, (const bf16_t*)delta, d_stride, w, (bf16_t*)y, n, eps);
  return 0;
}

VPSA_EXPORT int vpsa_glu_act(const void* x, long x_stride, void* y, int rows, int inter, int kind, int dtype,
                             hipStream_t st) {
  const long total = (long)rows * inter;
  if (total <= 0) return 0;
  if (kind < 0 || kind > 1) return -1;
  DISPATCH(dtype,
           hipLaunchKernelGGL(glu_act_kernel<bf16_t>, dim3(flat_grid(total)), dim3(256), 0, st, (const bf16_t*)x, x_stride, (bf16_t*)y, inter, total, kind),
           hipLaunchKernelGGL(glu_act_kernel<float>, dim3(flat_grid(total)), dim3(256), 0, st, (const float*)x, x_stride, (float*)y, inter, total, kind));
  return 0;
}

VPSA_EXPORT int vpsa_gather_rows(const void* x, const int* idx, void* xs, int rows, int n, int dtype,
                                 hipStream_t st) {
  if (rows <= 0) return 0;
  DISPATCH(dtype,
           hipLaunchKernelGGL(gather_rows_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (const bf16_t*)x, idx, (bf16_t*)xs, n),
           hipLaunchKernelGGL(gather_rows_kernel<float>, dim3(rows), dim3(256), 0, st, (const float*)x, idx, (float*)xs, n));
  return 0;
}

VPSA_EXPORT int vpsa_moe_finish(float* residual, const void* y, const float* weights, const int* pos, int topk,
                                const void* shared, const float* gate, int tokens, int n, int overwrite, int dtype,
                                hipStream_t st) {
  if (tokens <= 0) return 0;
  DISPATCH(dtype,
           hipLaunchKernelGGL(moe_finish_kernel<bf16_t>, dim3(tokens), dim3(256), 0, st, residual, (const bf16_t*)y, weights, pos, topk, (const bf16_t*)shared, gate, n, overwrite),
           hipLaunchKernelGGL(moe_finish_kernel<float>, dim3(tokens), dim3(256), 0, st, residual, (const float*)y, weights, pos, topk, (const float*)shared, gate, n, overwrite));
  return 0;
}
