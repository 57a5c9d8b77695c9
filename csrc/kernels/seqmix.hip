// Sequence mixers with carried state, for gfx950: linear-attention recurrences (fixed decay per head, or a
// forget gate per channel whose complement is the write strength), a short causal convolution in front of a
// windowed softmax attention with kept first tokens, capped scores, a sink and post-softmax head mixing,
// the Dynamic Tanh norm on a 32-bit residual stream, and the xIELU activation.  bf16 or fp32 activations
// (dtype 0 / 1 in the entry points); norms, angles, gates, decays, recurrent state, scores and softmax
// weights are fp32 in both.
//
//   add_dyt            residual += s1 d1 + s2 d2;  y = tanh(alpha residual) w + b
//   recurrent_scan     per (sequence, head): S <- a_t (.) S + k_t v_t^T,  o_t = S^T q_t, state in registers,
//                      carried in a per-sequence fp32 slot (zero when the chunk starts at position 0); the fixed-decay
//                      form optionally on silu(q), silu(k), silu(v)
//   head_rms           o[t, h, :] / rms(o[t, h, :]) (* w) (* silu(gate[t, h, :]))
//   short_conv_qkv     y_t = sum_j w[:, j] u_(t - taps + 1 + j) over a sequence's projected rows (the rows
//                      before the chunk come from the sequence's slot), rotary q / k, k and v -> paged cache
//   conv_tail          the last taps - 1 projected rows of every sequence -> its slot
//   window_attention   softmax(cap tanh(q k scale / cap)) with a sink in the denominator over the keys
//                      j <= i with i - j < window or j < keep_first (or: of i's own chunk of positions; or: of the
//                      window and one pooled entry per block of tokens before it), applied to the values of EVERY
//                      KV head or of the head's own
//   mix_heads          out[t, h] = sum_g talk[h, g] u[t, g, kv_head(h)]
//   xielu              z > 0: a_p z^2 + z / 2;  else a_n (exp(z) - 1 - z) + z / 2
//   qk_norm_write      q and k heads to unit root mean square (a weight per channel, a rotation of the first
//                      channels where given), q times a temperature that grows with the logarithm of the position,
//                      k and v -> paged cache (the layout window_attention reads; value heads may be fewer than key heads)
//   pool_blocks        mean key and mean value of every block of P tokens a step completes -> the pooled region of
//                      the sequence's pages (window_attention with pool > 0 sees the blocks before its window)
//   diff_heads         a1 - lambda a2 of a differential attention's two maps, unit root mean square, a factor
//   gla_prepare        q scale | k | sigmoid(z + b)^(1 / tau) per key channel, for prepared_scan
//   mlstm_gates        capped exponential input / forget gates of a matrix memory with their running maximum
//                      (carried per sequence and head), turned into one decay and one write strength per token
//   mlstm_prepare      q scale | k * write strength | decay, for prepared_scan
//   prepared_scan      recurrent_scan on rows prepared by the caller; optionally one more value column of ones,
//                      whose read-out is the normaliser's dot product with the query
//   head_finish        head_rms with its parts optional: stabilised division by the normaliser column, unit RMS,
//                      a weight per channel or per head and channel, a silu or sigmoid gate (a workgroup per head
//                      from a thousand channels on)
//
// Plain kernels: every size is taken (bounds below are checked by the entry points).
#include "common.h"
#include <stdlib.h>

namespace {

template <typename T> struct Cv;
template <> struct Cv<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Cv<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return (float)*p; }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = (bf16_t)v; }
  static __device__ __forceinline__ float round(float v) { return (float)(bf16_t)v; }
};

__device__ __forceinline__ float blk_sum(float v, float* red) {
  v = wave_reduce_sum(v);
  const int tid = threadIdx.x;
  __syncthreads();
  if ((tid & 63) == 0) red[tid >> 6] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) s += red[i];
  return s;
}

__device__ __forceinline__ float blk_max(float v, float* red) {
  v = wave_reduce_max(v);
  const int tid = threadIdx.x;
  __syncthreads();
  if ((tid & 63) == 0) red[tid >> 6] = v;
  __syncthreads();
  float s = red[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) s = fmaxf(s, red[i]);
  return s;
}

__device__ __forceinline__ float sigm(float x) { return 1.f / (1.f + expf(-x)); }

// Channel i of a head after the rotation of its first `dims` channels; x(c) reads channel c, cs is the
// table row of the token's position (cos[0 .. dims/2) | sin[0 .. dims/2)).  layout 0 pairs channel c with
// c + dims/2, layout 1 pairs 2c with 2c + 1.
template <typename F>
__device__ __forceinline__ float rotated(F x, int i, const float* __restrict__ cs, int dims, int layout) {
  if (i >= dims) return x(i);
  const int half = dims >> 1;
  if (layout == 0) {
    if (i < half) return x(i) * cs[i] - x(i + half) * cs[half + i];
    return x(i) * cs[i - half] + x(i - half) * cs[i];
  }
  const int p = i >> 1;
  if ((i & 1) == 0) return x(i) * cs[p] - x(i + 1) * cs[half + p];
  return x(i) * cs[p] + x(i - 1) * cs[half + p];
}

// ---------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void add_dyt_kernel(float* __restrict__ residual, const T* __restrict__ d1, long s1,
                                                      float c1, const T* __restrict__ d2, long s2, float c2,
                                                      const float* __restrict__ w, const float* __restrict__ b,
                                                      const float* __restrict__ alpha, T* __restrict__ y, int n) {
  const long row = blockIdx.x;
  float* r = residual + row * n;
  const float a = alpha[0];
  for (int i = threadIdx.x; i < n; i += 256) {
    float v = r[i];
    if (d1) v += c1 * Cv<T>::ld(d1 + row * s1 + i);
    if (d2) v += c2 * Cv<T>::ld(d2 + row * s2 + i);
    if (d1 || d2) r[i] = v;
    if (y) Cv<T>::st(y + row * (long)n + i, tanhf(a * v) * w[i] + b[i]);
  }
}

// ---------------------------------------------------------------------------------
// What enters a recurrence besides v, in fp32: prep [rows, heads, NP, dim] = q' | k' (| a).
// Fixed decay (NP = 2): q and k rotated by the position's table row, k times k_scale.
// Gated (NP = 3): q' = silu(q), a = lower + (1 - lower) sigmoid(logit + bias), k' = 1 - a.
template <typename T, bool GATED>
__global__ __launch_bounds__(256) void scan_prepare_kernel(const T* __restrict__ proj, long p_stride, int q_col, int k_col,
                                                           int heads, int dim, const int* __restrict__ positions,
                                                           const float* __restrict__ cos_sin, int rot_dims, int layout,
                                                           float k_scale, const float* __restrict__ gate_bias,
                                                           const float* __restrict__ gate_lower,
                                                           float* __restrict__ prep, int qk_act) {
  // qk_act (fixed decay): q and k pass through silu before the rotation
  constexpr int NP = GATED ? 3 : 2;
  const long row = blockIdx.x;
  const T* qp = proj + row * p_stride + q_col;
  const T* kp = proj + row * p_stride + k_col;
  float* dst = prep + row * (long)heads * NP * dim;
  const float* cs = GATED ? nullptr : cos_sin + (long)positions[row] * rot_dims;
  for (int e = threadIdx.x; e < heads * dim; e += 256) {
    const int h = e / dim, i = e - h * dim;
    float* d = dst + (long)h * NP * dim + i;
    if (GATED) {
      const float x = Cv<T>::ld(qp + e);
      const float lo = gate_lower[e];
      const float a = lo + (1.f - lo) * sigm(Cv<T>::ld(kp + e) + gate_bias[e]);
      d[0] = x * sigm(x);
      d[dim] = 1.f - a;
      d[2 * dim] = a;
    } else {
      const T* qh = qp + h * dim;
      const T* kh = kp + h * dim;
      auto act = [&](float x) { return qk_act ? x * sigm(x) : x; };
      d[0] = rotated([&](int c) { return act(Cv<T>::ld(qh + c)); }, i, cs, rot_dims, layout);
      d[dim] = rotated([&](int c) { return act(Cv<T>::ld(kh + c)); }, i, cs, rot_dims, layout) * k_scale;
    }
  }
}

// ---------------------------------------------------------------------------------
// The recurrence S <- a_t (.) S + k_t v_t^T, o_t = S^T q_t with the state in registers.  A thread holds a tile
// of RPT rows x 4 columns of S; a column group's `dim` rows are spread over R neighbouring lanes (row
// i = j * R + lane group), a workgroup covers 1024 / R columns of one head.  A block of up to TB tokens is
// prepared in LDS (rotation or gates, fp32), then walked token by token.
//
// PHASE 0: whole sequences, from and to their state slots (decode rows, short chunks).
// Long chunks are cut into pieces that run side by side (the recurrence is linear in S):
// PHASE 1: a piece's end state from zero (no outputs) -> ws_state[piece];
//          scan_propagate_kernel then walks a sequence's pieces, S <- A_piece (.) S + end state, leaves every
//          piece's START state in ws_state and the sequence's end state in its slot;
// PHASE 2: a piece's outputs from its start state.
template <typename T, int RPT, bool GATED, bool FOLD, int PHASE>
__global__ __launch_bounds__(256) void recurrent_scan_kernel(
    const T* __restrict__ proj, long p_stride, int v_col, int heads, int dim, int vdim, const float* __restrict__ prep,
    float* __restrict__ state, long state_stride, const int* __restrict__ seq_cu, const int* __restrict__ seq_state,
    const int* __restrict__ positions, const float* __restrict__ decay, float* __restrict__ out, int R, int TB,
    const int* __restrict__ pieces, float* __restrict__ ws_state, int vsrc, int unit_col, int v_act) {
  // v_act: values pass through silu on their way in
  // vsrc: value columns per head that `proj` holds (vdim, or one less than the state's columns need when
  // unit_col: column vsrc of every token's value is then 1 and columns past it are 0)
  constexpr int NP = GATED ? 3 : 2;
  extern __shared__ float smem[];
  const int head = blockIdx.y;
  int seq, r0, r1;
  if (PHASE == 0) {
    seq = blockIdx.z, r0 = seq_cu[seq], r1 = seq_cu[seq + 1];
  } else {
    const int* pc = pieces + 3 * blockIdx.z;
    seq = pc[0], r0 = pc[1], r1 = pc[1] + pc[2];
  }
  const int slot = seq_state[seq];
  const int dimp = R * RPT, cols = (256 / R) * 4;
  const int tid = threadIdx.x, rg = tid % R, cb = tid / R;
  const int col = blockIdx.x * cols + cb * 4;
  if (slot < 0) {  // rows of no sequence (a padded batch): their output is zero
    if (PHASE != 1 && rg == 0)
      for (int r = r0; r < r1; ++r)
        for (int c = col; c < min(col + 4, vdim); ++c) out[((long)r * heads + head) * vdim + c] = 0.f;
    return;
  }
  if (r1 <= r0) return;
  float* qs = smem;
  float* ks = qs + TB * dimp;
  float* as = ks + TB * dimp;                       // gates (GATED only)
  float* vs = GATED ? as + TB * dimp : as;
  float* st = PHASE == 0 ? state + (long)slot * state_stride + (long)head * dim * vdim
                         : ws_state + ((long)blockIdx.z * heads + head) * dim * vdim;
  const bool vec = (vdim & 3) == 0 && (reinterpret_cast<uintptr_t>(st) & 15) == 0;  // whole, aligned float4 columns
  const bool fresh = PHASE == 1 || (PHASE == 0 && positions[r0] == 0);
  float S[RPT][4];
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const int i = ((j >> 2) * R + rg) * 4 + (j & 3);
#pragma unroll
    for (int c = 0; c < 4; ++c) S[j][c] = 0.f;
    if (!fresh && i < dim) {
      if (vec && col < vdim) {
        const f32x4 v4 = *reinterpret_cast<const f32x4*>(st + (long)i * vdim + col);
#pragma unroll
        for (int c = 0; c < 4; ++c) S[j][c] = v4[c];
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (col + c < vdim) S[j][c] = st[(long)i * vdim + col + c];
      }
    }
  }
  const float dec = GATED ? 0.f : decay[head];
  // A fixed decay is folded into the staged block: with S~_t = S_t / dec^(t+1) inside a block of TB tokens the
  // update is one multiply-add, S~_t = S~_(t-1) + (k_t / dec^(t+1)) v_t^T, the read-out another,
  // o_t = S~_t^T (dec^(t+1) q_t), and the block ends with S = S~ dec^nb.  (Two operations per state element and
  // token instead of three.)  Decays whose TB-th power leaves fp32's comfortable range take the plain form (FOLD off).
  constexpr bool folded = FOLD && !GATED;  // the caller checks the decays (dec^TB well inside fp32's range)
  if (dimp > dim)  // rows past the head's size stay zero in every staged block
    for (int e = tid; e < TB * NP * dimp; e += 256) smem[e] = 0.f;
  for (int rb = r0; rb < r1; rb += TB) {
    const int nb = min(TB, r1 - rb);
    __syncthreads();
    for (int e = tid; e < nb * NP * dim; e += 256) {  // prepared rows are contiguous per (row, head)
      const int tt = e / (NP * dim), rem = e - tt * (NP * dim);
      const int which = rem / dim, i = rem - which * dim;
      if (PHASE == 1 && which == 0) continue;         // no outputs: no queries
      float x = prep[((long)(rb + tt) * heads + head) * NP * dim + rem];
      if (folded) {
        float pw = dec;
        for (int t = 0; t < tt; ++t) pw *= dec;       // dec^(tt + 1)
        x = which == 0 ? x * pw : x / pw;
      }
      (which == 0 ? qs : which == 1 ? ks : as)[tt * dimp + i] = x;
    }
    for (int e = tid; e < nb * cols; e += 256) {
      const int tt = e / cols, c = e - tt * cols;
      const int cc = blockIdx.x * cols + c;
      float x = cc < vsrc ? Cv<T>::ld(proj + (long)(rb + tt) * p_stride + v_col + head * vsrc + cc)
                          : ((unit_col && cc == vsrc) ? 1.f : 0.f);
      if (v_act) x = x * sigm(x);
      vs[e] = x;
    }
    __syncthreads();
    // a wave whose columns all lie past the state's (the last column block of a width that is no multiple of the
    // block) only helps to stage: its lanes hold zeros that nobody reads
    if (blockIdx.x * cols + (tid >> 6) * (64 / R) * 4 >= vdim) continue;
    for (int tt = 0; tt < nb; ++tt) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(vs + tt * cols + cb * 4);
      const float* qr = qs + tt * dimp + rg * 4;
      const float* kr = ks + tt * dimp + rg * 4;
      const float* ar = as + tt * dimp + rg * 4;
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int jg = 0; jg < RPT / 4; ++jg) {  // four rows per 16-byte LDS read
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(kr + jg * R * 4);
        f32x4 q4 = {0.f, 0.f, 0.f, 0.f}, a4 = {dec, dec, dec, dec};
        if (PHASE != 1) q4 = *reinterpret_cast<const f32x4*>(qr + jg * R * 4);
        if (GATED) a4 = *reinterpret_cast<const f32x4*>(ar + jg * R * 4);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int j = jg * 4 + jj;
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            S[j][c] = folded ? fmaf(k4[jj], v[c], S[j][c]) : fmaf(a4[jj], S[j][c], k4[jj] * v[c]);
            if (PHASE != 1) acc[c] = fmaf(S[j][c], q4[jj], acc[c]);
          }
        }
      }
      if (folded && tt == nb - 1) {  // back to the true state at the block's end
        float pw = 1.f;
        for (int t = 0; t < nb; ++t) pw *= dec;
#pragma unroll
        for (int j = 0; j < RPT; ++j)
#pragma unroll
          for (int c = 0; c < 4; ++c) S[j][c] *= pw;
      }
      if (PHASE != 1) {
        // (DPP adds instead of these shuffles were measured: 1.31 -> 1.46 ms per 8192 rows, their wait states sit
        // on the chain from the last multiply-add to the store)
        for (int off = R >> 1; off > 0; off >>= 1) {
#pragma unroll
          for (int c = 0; c < 4; ++c) acc[c] += __shfl_xor(acc[c], off, 64);
        }
        if (rg == 0) {
          float* op = out + ((long)(rb + tt) * heads + head) * vdim + col;
          if ((vdim & 3) == 0 && col < vdim) *reinterpret_cast<f32x4*>(op) = (f32x4){acc[0], acc[1], acc[2], acc[3]};
          else
            for (int c = 0; c < 4; ++c)
              if (col + c < vdim) op[c] = acc[c];
        }
      }
    }
  }
  if (PHASE == 2) return;
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const int i = ((j >> 2) * R + rg) * 4 + (j & 3);
    if (i >= dim) continue;
    if (vec && col < vdim) {
      *reinterpret_cast<f32x4*>(st + (long)i * vdim + col) = (f32x4){S[j][0], S[j][1], S[j][2], S[j][3]};
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (col + c < vdim) st[(long)i * vdim + col + c] = S[j][c];
    }
  }
}

// A piece's total decay per state row, prod_t a_t[i] -> ws_decay[piece][head][i].  One workgroup per (piece, head).
template <typename T, bool GATED>
__global__ __launch_bounds__(128) void scan_decay_kernel(const T* __restrict__ proj, long p_stride, int k_col, int heads,
                                                         int dim, const float* __restrict__ decay,
                                                         const float* __restrict__ gate_bias,
                                                         const float* __restrict__ gate_lower,
                                                         const int* __restrict__ pieces, float* __restrict__ ws_decay) {
  const int piece = blockIdx.x, head = blockIdx.y;
  const int r0 = pieces[3 * piece + 1], n = pieces[3 * piece + 2];
  for (int i = threadIdx.x; i < dim; i += 128) {
    float p = 1.f;
    if (GATED) {
      const float lo = gate_lower[head * dim + i], b = gate_bias[head * dim + i];
      for (int r = r0; r < r0 + n; ++r)
        p *= lo + (1.f - lo) * sigm(Cv<T>::ld(proj + (long)r * p_stride + k_col + head * dim + i) + b);
    } else {
      const float d = decay[head];
      for (int r = 0; r < n; ++r) p *= d;
    }
    ws_decay[((long)piece * heads + head) * dim + i] = p;
  }
}

// Walks a sequence's pieces in order: ws_state[piece] (the piece's end state from zero) becomes its START
// state, and the sequence's slot gets the end state.  One thread per state element.
__global__ __launch_bounds__(256) void scan_propagate_kernel(float* __restrict__ ws_state, const float* __restrict__ ws_decay,
                                                             float* __restrict__ state, long state_stride,
                                                             const int* __restrict__ seq_cu,
                                                             const int* __restrict__ seq_state,
                                                             const int* __restrict__ seq_pieces,
                                                             const int* __restrict__ positions, int heads, int dim,
                                                             int vdim) {
  const int seq = blockIdx.z, head = blockIdx.y;
  const int slot = seq_state[seq];
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (slot < 0 || e >= dim * vdim || seq_cu[seq + 1] <= seq_cu[seq]) return;
  const int i = e / vdim;
  float* st = state + (long)slot * state_stride + (long)head * dim * vdim + e;
  float S = positions[seq_cu[seq]] == 0 ? 0.f : *st;
  for (int pc = seq_pieces[seq]; pc < seq_pieces[seq + 1]; ++pc) {
    float* w = ws_state + ((long)pc * heads + head) * dim * vdim + e;
    const float end = *w;
    *w = S;
    S = fmaf(ws_decay[((long)pc * heads + head) * dim + i], S, end);
  }
  *st = S;
}

// A piece's total decay per state row from prepared rows (prep [rows, heads, 3, dim], the third part).
__global__ __launch_bounds__(128) void scan_decay_prep_kernel(const float* __restrict__ prep, int heads, int dim,
                                                              const int* __restrict__ pieces,
                                                              float* __restrict__ ws_decay) {
  const int piece = blockIdx.x, head = blockIdx.y;
  const int r0 = pieces[3 * piece + 1], n = pieces[3 * piece + 2];
  for (int i = threadIdx.x; i < dim; i += 128) {
    float p = 1.f;
    for (int r = r0; r < r0 + n; ++r) p *= prep[((long)r * heads + head) * 3 * dim + 2 * dim + i];
    ws_decay[((long)piece * heads + head) * dim + i] = p;
  }
}

__device__ __forceinline__ float log_sigm(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// Gated linear attention: prep = q * q_scale | k | a,  a = sigmoid(z + b)^(1 / tau) per head and key channel.
template <typename T>
__global__ __launch_bounds__(256) void gla_prepare_kernel(const T* __restrict__ proj, long p_stride, int q_col, int k_col,
                                                          const T* __restrict__ z, long z_stride,
                                                          const float* __restrict__ z_bias, int heads, int dim,
                                                          float q_scale, float inv_tau, float* __restrict__ prep) {
  const long row = blockIdx.x;
  const T* pr = proj + row * p_stride;
  float* dst = prep + row * (long)heads * 3 * dim;
  for (int e = threadIdx.x; e < heads * dim; e += 256) {
    const int h = e / dim, i = e - h * dim;
    float* d = dst + (long)h * 3 * dim + i;
    d[0] = Cv<T>::ld(pr + q_col + e) * q_scale;
    d[dim] = Cv<T>::ld(pr + k_col + e);
    d[2 * dim] = expf(log_sigm(Cv<T>::ld(z + row * z_stride + e) + z_bias[e]) * inv_tau);
  }
}

// Matrix memory with exponential gates.  Per head and token a log input gate i = cap tanh((x_i + b_i) / cap) and a
// log forget gate f = logsigmoid(cap tanh((x_f + b_f) / cap)); a running maximum m_t = max(f_t + m_(t-1), i_t)
// (m = 0 before the first token) keeps the exponentials in range:
//   decay_t = exp(f_t + m_(t-1) - m_t),  write_t = exp(i_t - m_t).
// The map m -> max(a + m, b) composes associatively, so a wave scans 64 tokens per step.  m is carried in the
// sequence's state slot.  logits fp32 [rows, 2 heads] = x_i | x_f.  One wave per (sequence, head).
__global__ __launch_bounds__(64) void mlstm_gates_kernel(const float* __restrict__ logits, const float* __restrict__ bias_i,
                                                         const float* __restrict__ bias_f, float cap, int heads,
                                                         float* __restrict__ state, long state_stride,
                                                         const int* __restrict__ seq_cu,
                                                         const int* __restrict__ seq_state,
                                                         const int* __restrict__ positions, float* __restrict__ ab,
                                                         float* __restrict__ mrow) {
  const int seq = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int r0 = seq_cu[seq], r1 = seq_cu[seq + 1];
  const int slot = seq_state[seq];
  if (r1 <= r0) return;
  if (slot < 0) {  // rows of no sequence: nothing is written into a state, the read-out is zero
    for (int r = r0 + lane; r < r1; r += 64) {
      ab[((long)r * heads + head) * 2] = 0.f;
      ab[((long)r * heads + head) * 2 + 1] = 0.f;
      mrow[(long)r * heads + head] = 0.f;
    }
    return;
  }
  float* mp = state + (long)slot * state_stride + head;
  float m0 = positions[r0] == 0 ? 0.f : *mp;
  const float bi = bias_i[head], bf = bias_f[head];
  for (int rb = r0; rb < r1; rb += 64) {
    const int r = rb + lane;
    const bool live = r < r1;
    float gi = -INFINITY, gf = 0.f;
    if (live) {
      gi = cap * tanhf((logits[(long)r * 2 * heads + head] + bi) / cap);
      gf = log_sigm(cap * tanhf((logits[(long)r * 2 * heads + heads + head] + bf) / cap));
    }
    float a = gf, b = gi;  // this token's map, then the composition of all maps up to it
    for (int off = 1; off < 64; off <<= 1) {
      const float pa = __shfl_up(a, off, 64), pb = __shfl_up(b, off, 64);
      if (lane >= off) {
        b = fmaxf(pb + a, b);
        a = pa + a;
      }
    }
    const float m = fmaxf(a + m0, b);
    float prev = __shfl_up(m, 1, 64);
    if (lane == 0) prev = m0;
    if (live) {
      ab[((long)r * heads + head) * 2] = expf(gf + prev - m);
      ab[((long)r * heads + head) * 2 + 1] = expf(gi - m);
      mrow[(long)r * heads + head] = m;
    }
    m0 = __shfl(m, min(63, r1 - rb - 1), 64);
  }
  if (lane == 0) *mp = m0;
}

// prep = q * q_scale | k * write | decay (one decay for all key channels of a head)
template <typename T>
__global__ __launch_bounds__(256) void mlstm_prepare_kernel(const T* __restrict__ proj, long p_stride, int q_col,
                                                            int k_col, const float* __restrict__ ab, int heads, int dim,
                                                            float q_scale, float* __restrict__ prep) {
  const long row = blockIdx.x;
  const T* pr = proj + row * p_stride;
  float* dst = prep + row * (long)heads * 3 * dim;
  for (int e = threadIdx.x; e < heads * dim; e += 256) {
    const int h = e / dim, i = e - h * dim;
    float* d = dst + (long)h * 3 * dim + i;
    const float dec = ab[(row * heads + h) * 2], wr = ab[(row * heads + h) * 2 + 1];
    d[0] = Cv<T>::ld(pr + q_col + e) * q_scale;
    d[dim] = Cv<T>::ld(pr + k_col + e) * wr;
    d[2 * dim] = dec;
  }
}

// A workgroup per row, a wave per head in turn.  Row = q [heads * dim] (| k [kv_heads * dim] | v [v_heads * vdim]
// when the layer owns its cache entries).  q and k heads are divided by their root mean square (eps inside the
// root), multiplied by a weight per channel where one is given (qw / kw, shared by the heads), and turned by the
// rotary table over their first rot_dims channels (cos_sin null: no rotation); q is then multiplied by
// 1 + coef ln(floor((p + 1) / every) + 1) at position p.  k and v go to the page layout of window_attention
// (K key by key, V transposed); designs with several key maps per value head have fewer value heads than key heads.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_write_kernel(const T* __restrict__ proj, long p_stride, int heads,
                                                            int kv_heads, int dim, int vdim, int own,
                                                            const int* __restrict__ positions,
                                                            const long* __restrict__ slots, float eps, float coef,
                                                            float every, T* __restrict__ q_out, T* __restrict__ cache,
                                                            long page_stride, int v_heads,
                                                            const float* __restrict__ qw, const float* __restrict__ kw,
                                                            const float* __restrict__ cos_sin, int rot_dims,
                                                            int layout) {
  const long row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* pr = proj + row * p_stride;
  const int p = positions[row];
  float temp = 1.f;
  if (coef != 0.f) temp = 1.f + coef * logf((float)floor((double)(p + 1) / (double)every) + 1.f);
  const long slot = own ? slots[row] : -1;
  const int nk = kv_heads * dim;
  // (a few rows per launch: the heads are spread over blockIdx.y; many rows: one workgroup walks them in turn)
  for (int hh = blockIdx.y * 4 + wave; hh < heads + (own ? kv_heads : 0); hh += gridDim.y * 4) {
    const T* src = pr + (long)hh * dim;  // k heads follow the q heads
    float ss = 0.f;
    for (int i = lane; i < dim; i += 64) {
      const float v = Cv<T>::ld(src + i);
      ss += v * v;
    }
    ss = wave_reduce_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)dim + eps);
    const float* w = hh < heads ? qw : kw;
    const float* cs = cos_sin ? cos_sin + (long)p * rot_dims : nullptr;
    auto normed = [&](int c) { return Cv<T>::ld(src + c) * inv * (w ? w[c] : 1.f); };
    auto value = [&](int i) { return cs ? rotated(normed, i, cs, rot_dims, layout) : normed(i); };
    if (hh < heads) {
      for (int i = lane; i < dim; i += 64) Cv<T>::st(q_out + (row * heads + hh) * dim + i, value(i) * temp);
    } else if (slot >= 0) {
      T* dst = cache + (slot / PAGE) * page_stride + (slot % PAGE) * nk + (long)(hh - heads) * dim;
      for (int i = lane; i < dim; i += 64) Cv<T>::st(dst + i, value(i));
    }
  }
  if (slot >= 0) {
    const T* vs = pr + (long)heads * dim + nk;
    T* dst = cache + (slot / PAGE) * page_stride + (long)PAGE * nk + (slot % PAGE);
    for (int c = blockIdx.y * 256 + threadIdx.x; c < v_heads * vdim; c += gridDim.y * 256) dst[(long)c * PAGE] = vs[c];
  }
}

// Pooled entries of a windowed attention that also sees a mean key and value per block of `pool` tokens.  A row
// of the step at position p with (p + 1) % pool == 0 completes block b = p / pool; the
// block's keys and values are read back from the pages (as the cache holds them, whichever step wrote them), summed
// in position order in fp32 and divided by pool, and stored as entry b % PAGE of the pooled region (pool_off
// elements behind the token region, same layout) of the sequence's page b / PAGE.
constexpr int POOL_ROWS = 16;  // rows of the step a workgroup looks at

template <typename T>
__global__ __launch_bounds__(256) void pool_blocks_kernel(T* __restrict__ cache, long page_stride, long pool_off,
                                                          const int* __restrict__ block_tables, int bt_stride,
                                                          const int* __restrict__ row_seq,
                                                          const int* __restrict__ positions,
                                                          const long* __restrict__ slots, int rows, int nk, int nv,
                                                          int pool) {
  // blockIdx.x: a run of POOL_ROWS rows, of which those that complete a block are worked on one after the other
  // (most workgroups find none or one); blockIdx.y: a run of 256 channels (keys first, then values).  A thread owns
  // one channel and walks the block's tokens page by page (a page's tokens are a strided run for a key channel, a
  // contiguous one for a value channel), summing in position order.
  __shared__ int todo[POOL_ROWS];
  const int tid = threadIdx.x;
  if (tid < POOL_ROWS) {
    const long row = (long)blockIdx.x * POOL_ROWS + tid;
    int p = -1;
    if (row < rows && slots[row] >= 0 && (positions[row] + 1) % pool == 0) p = positions[row];
    todo[tid] = p;
  }
  __syncthreads();
  const int c = blockIdx.y * 256 + tid;
  if (c >= nk + nv) return;
  const bool is_k = c < nk;
  const long off = is_k ? c : (long)PAGE * nk + (long)(c - nk) * PAGE, step = is_k ? nk : 1;
  for (int k = 0; k < POOL_ROWS; ++k) {
    const int p = todo[k];
    if (p < 0) continue;
    const long row = (long)blockIdx.x * POOL_ROWS + k;
    const int seq = row_seq ? row_seq[row] : (int)row;
    const int* bt = block_tables + (long)seq * bt_stride;
    const int b = p / pool, j0 = b * pool;
    float acc = 0.f;
    for (int pg = j0 / PAGE; pg <= p / PAGE; ++pg) {
      const int a = max(j0, pg * PAGE) % PAGE, e = min(p, pg * PAGE + PAGE - 1) % PAGE;
      const T* src = cache + (long)bt[pg] * page_stride + off;
#pragma unroll 8
      for (int r = a; r <= e; ++r) acc += Cv<T>::ld(src + r * step);
    }
    T* dst = cache + (long)bt[b / PAGE] * page_stride + pool_off + off;
    Cv<T>::st(dst + (b % PAGE) * step, acc / (float)pool);
  }
}

// Differential attention's combination.  u fp32 [rows, 2 heads, vdim]: per key/value group g of `rep` query heads the
// first map's outputs of its heads, then the second map's ([g][map][head in group]).  One wave per (row, head):
// o = a1 - lambda a2, divided by its root mean square over vdim (eps inside the root), times post; y [rows, heads * vdim]
// with the heads in their natural order.
template <typename T>
__global__ __launch_bounds__(256) void diff_heads_kernel(const float* __restrict__ u, T* __restrict__ y, long pairs,
                                                         int heads, int rep, int vdim, float lambda, float eps,
                                                         float post) {
  const long pair = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long row = pair / heads;
  const int head = (int)(pair - row * heads);
  const int g = head / rep, j = head - g * rep;
  const float* a1 = u + ((row * 2 * heads) + (long)g * 2 * rep + j) * vdim;
  const float* a2 = a1 + (long)rep * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += 64) {
    const float v = a1[c] - lambda * a2[c];
    ss += v * v;
  }
  ss = wave_reduce_sum(ss);
  const float inv = post / sqrtf(ss / (float)vdim + eps);
  for (int c = lane; c < vdim; c += 64) Cv<T>::st(y + pair * vdim + c, (a1[c] - lambda * a2[c]) * inv);
}

// One wave per (row, head).  o [pairs][ostride] fp32, of which the first vdim columns are the head's output.
// stab: column vdim of o is the normaliser's dot product with the query and stab[pair] the running maximum m of the
// gates: the output is first divided by max(|n . q|, exp(-m)) + 1e-6.  unit: divide by the root mean square over
// vdim (eps inside the root).  w: a weight per channel (w_heads 0: shared by the heads) or per head and channel.
// gate: times silu (gate_act 0) or sigmoid (1) of gate[row, head * vdim + c].
template <typename T>
__global__ __launch_bounds__(256) void head_rms_kernel(const float* __restrict__ o, int ostride,
                                                       const float* __restrict__ stab, int unit,
                                                       const float* __restrict__ w, int w_heads,
                                                       const T* __restrict__ gate, long g_stride, int gate_act,
                                                       T* __restrict__ y, long pairs, int heads, int vdim, float eps) {
  const long pair = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long row = pair / heads;
  const int head = (int)(pair - row * heads);
  const float* op = o + pair * ostride;
  float pre = 1.f;
  if (stab) pre = 1.f / (fmaxf(fabsf(op[vdim]), expf(-stab[pair])) + 1e-6f);
  float inv = 1.f;
  if (unit) {
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) {
      const float v = op[c] * pre;
      ss += v * v;
    }
    ss = wave_reduce_sum(ss);
    inv = 1.f / sqrtf(ss / (float)vdim + eps);
  }
  for (int c = lane; c < vdim; c += 64) {
    float v = op[c] * pre * inv;
    if (w) v *= w[w_heads ? head * vdim + c : c];
    if (gate) {
      const float g = Cv<T>::ld(gate + row * g_stride + head * vdim + c);
      v *= gate_act == 0 ? g * sigm(g) : sigm(g);
    }
    Cv<T>::st(y + pair * vdim + c, v);
  }
}

// The same with one workgroup per (row, head), for heads of a thousand channels and more (all heads of a mixer
// normed together, say), where a single wave per head would walk its channels alone.
template <typename T>
__global__ __launch_bounds__(256) void head_rms_wide_kernel(const float* __restrict__ o, int ostride,
                                                            const float* __restrict__ stab, int unit,
                                                            const float* __restrict__ w, int w_heads,
                                                            const T* __restrict__ gate, long g_stride, int gate_act,
                                                            T* __restrict__ y, int heads, int vdim, float eps) {
  __shared__ float red[4];
  const long pair = blockIdx.x;
  const long row = pair / heads;
  const int head = (int)(pair - row * heads);
  const float* op = o + pair * ostride;
  float pre = 1.f;
  if (stab) pre = 1.f / (fmaxf(fabsf(op[vdim]), expf(-stab[pair])) + 1e-6f);
  float inv = 1.f;
  if (unit) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < vdim; c += 256) {
      const float v = op[c] * pre;
      ss += v * v;
    }
    inv = 1.f / sqrtf(blk_sum(ss, red) / (float)vdim + eps);
  }
  for (int c = threadIdx.x; c < vdim; c += 256) {
    float v = op[c] * pre * inv;
    if (w) v *= w[w_heads ? head * vdim + c : c];
    if (gate) {
      const float g = Cv<T>::ld(gate + row * g_stride + head * vdim + c);
      v *= gate_act == 0 ? g * sigm(g) : sigm(g);
    }
    Cv<T>::st(y + pair * vdim + c, v);
  }
}

// ---------------------------------------------------------------------------------
// One workgroup per row.  chans = heads * dim + kv_heads * (dim + vdim) projected channels q | k | v.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_qkv_kernel(
    const T* __restrict__ proj, long p_stride, const float* __restrict__ conv_w, int taps, int heads, int kv_heads,
    int dim, int vdim, const float* __restrict__ state, long state_stride, const int* __restrict__ row_seq,
    const int* __restrict__ seq_cu, const int* __restrict__ seq_state, const int* __restrict__ positions,
    const long* __restrict__ slots, const float* __restrict__ cos_sin, int rot_dims, int layout, T* __restrict__ q_out,
    T* __restrict__ cache, long page_stride) {
  extern __shared__ float ys[];
  const long row = blockIdx.x;
  const int seq = row_seq ? row_seq[row] : (int)row;
  const int slot = seq_state[seq];
  const int r0 = seq_cu[seq];
  const int pos = positions[row], pos0 = positions[r0];
  const int chans = heads * dim + kv_heads * (dim + vdim);
  const float* tail = slot >= 0 ? state + (long)slot * state_stride : nullptr;
  for (int c = threadIdx.x; c < chans; c += 256) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      const long src = row - back;
      float u = 0.f;
      if (src >= r0) {
        u = Cv<T>::ld(proj + src * p_stride + c);
      } else if (pos - back >= 0 && tail) {
        u = tail[(long)(pos - back - (pos0 - (taps - 1))) * chans + c];
      }
      acc = fmaf(conv_w[(long)c * taps + j], u, acc);
    }
    ys[c] = Cv<T>::round(acc);
  }
  __syncthreads();
  const float* cs = cos_sin + (long)pos * rot_dims;
  const int nq = heads * dim, nk = kv_heads * dim, nv = kv_heads * vdim;
  const long kv_slot = slots[row];
  T* kdst = kv_slot >= 0 ? cache + (kv_slot / PAGE) * page_stride + (kv_slot % PAGE) * (long)nk : nullptr;
  T* vdst = kv_slot >= 0 ? cache + (kv_slot / PAGE) * page_stride + (long)PAGE * nk + (kv_slot % PAGE) : nullptr;  // V^T
  for (int c = threadIdx.x; c < chans; c += 256) {
    if (c < nq + nk) {
      const int base = c < nq ? (c / dim) * dim : nq + ((c - nq) / dim) * dim;
      const float* x = ys + base;
      const float r = rotated([&](int i) { return x[i]; }, c - base, cs, rot_dims, layout);
      if (c < nq) Cv<T>::st(q_out + row * nq + c, r);
      else if (kdst) Cv<T>::st(kdst + (c - nq), r);
    } else if (vdst) {
      Cv<T>::st(vdst + (long)(c - nq - nk) * PAGE, ys[c]);
    }
  }
}

// One workgroup per sequence, after the convolution of the step: tail[j] = projected row of position
// end - (taps - 1) + j, from the chunk or, for chunks shorter than the tail, from the old tail (shifted:
// a thread owns a channel and walks j upwards, so it reads tail[j + n] before writing it).
template <typename T>
__global__ __launch_bounds__(256) void conv_tail_kernel(const T* __restrict__ proj, long p_stride, int taps, int chans,
                                                        float* __restrict__ state, long state_stride,
                                                        const int* __restrict__ seq_cu, const int* __restrict__ seq_state,
                                                        const int* __restrict__ positions) {
  const int seq = blockIdx.x;
  const int slot = seq_state[seq];
  const int r0 = seq_cu[seq], r1 = seq_cu[seq + 1];
  if (slot < 0 || r1 <= r0) return;
  const int n = r1 - r0, pos0 = positions[r0], keep = taps - 1;
  float* tail = state + (long)slot * state_stride;
  for (int c = threadIdx.x; c < chans; c += 256) {
    for (int j = 0; j < keep; ++j) {
      const int k = n + j - keep;  // chunk row of tail entry j (negative: before the chunk)
      float u = 0.f;
      if (k >= 0) u = Cv<T>::ld(proj + (long)(r0 + k) * p_stride + c);
      else if (pos0 + k >= 0) u = tail[(long)(j + n) * chans + c];
      tail[(long)j * chans + c] = u;
    }
  }
}

// ---------------------------------------------------------------------------------
// Layer cache inside a page: K [PAGE][kv_heads * dim], then V transposed [kv_heads * vdim][PAGE].
// The pages a query at position p (or a tile of queries p_a .. p_b) has to visit: those that hold kept first
// tokens below the window, then the window's own; the mask decides key by key.
// mode 1: `window` is a chunk size instead, and a query sees the keys of its own chunk (chunks counted from
// position 0) up to itself.
// pool > 0: beside its window a query at position p sees one pooled entry per block of `pool` tokens that lies
// wholly before the window, blocks 0 .. seen_blocks(p) - 1.  Block b's entry is entry b % PAGE of the pooled region
// of the sequence's page b / PAGE (same layout as the token region, pool_off elements behind it); the walk visits
// those pages first (its first n_keep visits, `pooled`), then the window's.  keep_first is 0 then.
__device__ __forceinline__ int seen_blocks(int p, int window, int pool) {
  const int a = p - window + 1;  // tokens before the window
  return a > 0 ? a / pool : 0;
}

struct PageWalk {
  int n_keep, first, count;
  bool pool_walk;
  __device__ __forceinline__ PageWalk(int pa, int pb, int window, int keep_first, int mode = 0, int pool = 0) {
    const int lo = mode == 1 ? pa - pa % window : max(0, pa - window + 1);
    first = lo / PAGE;
    pool_walk = pool > 0;
    if (pool_walk) n_keep = (seen_blocks(pb, window, pool) + PAGE - 1) / PAGE;
    else n_keep = min((min(keep_first, lo) + PAGE - 1) / PAGE, first);
    count = n_keep + pb / PAGE - first + 1;
  }
  __device__ __forceinline__ int page(int i) const { return i < n_keep ? i : first + (i - n_keep); }
  __device__ __forceinline__ bool pooled(int i) const { return pool_walk && i < n_keep; }
};

__device__ __forceinline__ bool key_seen(int j, int p, int window, int keep_first, int mode = 0) {
  if (mode == 1) return j <= p && j >= p - p % window;
  return j <= p && (p - j < window || j < keep_first);
}

// Plain kernel, every size and both dtypes.  One workgroup per (row, query head), four pages per step: a thread
// scores one key, then owns value channels and walks the step's keys in runs of 16 bytes.
// out [rows, heads, kv_heads, vdim] fp32: the head's softmax weights applied to the values of every KV head
// (the head mixing that follows needs them).
constexpr int WA_KEYS = 256;
constexpr int WA_ACC = 8;  // kv_heads * vdim <= 256 * WA_ACC

template <typename T>
__global__ __launch_bounds__(256) void window_attention_kernel(
    const T* __restrict__ q, long q_stride, const T* __restrict__ cache, long page_stride,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ row_seq,
    const int* __restrict__ positions, const float* __restrict__ sink, float* __restrict__ out, int heads, int kv_heads,
    int dim, int vdim, int window, int keep_first, float scale, float softcap, int own, int mode, int pool,
    long pool_off, int maps) {
  // own: only the values of the head's own KV head (out [rows, heads, vdim]); designs without head mixing
  // maps: key heads per value head (kv_heads counts key heads; key head g reads the values of head g / maps)
  extern __shared__ float sm[];
  __shared__ float red[4];
  __shared__ float ps[WA_KEYS];
  __shared__ long pbase[WA_KEYS / PAGE];
  constexpr int RUN = 16 / sizeof(T);  // keys per 16-byte load of a V^T row
  const long row = blockIdx.x;
  const int head = blockIdx.y;
  const int tid = threadIdx.x;
  const int seq = row_seq ? row_seq[row] : (int)row;
  const int pos = positions[row];
  const int g = head / (heads / kv_heads);
  const int nk = kv_heads * dim, nv = own ? vdim : kv_heads / maps * vdim;
  const int c0 = own ? g / maps * vdim : 0;  // first value channel this head reads
  const int nb = pool > 0 ? seen_blocks(pos, window, pool) : 0;
  float* qs = sm;
  for (int i = tid; i < dim; i += 256) qs[i] = Cv<T>::ld(q + row * q_stride + head * dim + i);
  const PageWalk walk(pos, pos, window, keep_first, mode, pool);
  const int* bt = block_tables + (long)seq * bt_stride;
  float m = sink ? sink[head] : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[WA_ACC];
#pragma unroll
  for (int a = 0; a < WA_ACC; ++a) acc[a] = 0.f;
  __syncthreads();
  for (int p0 = 0; p0 < walk.count; p0 += WA_KEYS / PAGE) {
    const int pi = p0 + tid / PAGE, r = tid % PAGE;
    float s = -INFINITY;
    if (pi < walk.count) {
      const int pg = walk.page(pi);
      const bool pooled = walk.pooled(pi);
      const long base = (long)bt[pg] * page_stride + (pooled ? pool_off : 0);
      if (r == 0) pbase[tid / PAGE] = base;
      const int j = pg * PAGE + r;
      if (pooled ? j < nb : key_seen(j, pos, window, keep_first, mode)) {
        const T* kp = cache + base + (long)r * nk + g * dim;
        float d = 0.f;
        for (int i = 0; i < dim; ++i) d = fmaf(qs[i], Cv<T>::ld(kp + i), d);
        d *= scale;
        s = softcap > 0.f ? softcap * tanhf(d / softcap) : d;
      }
    }
    const float mb = blk_max(s, red);
    const float mn = fmaxf(m, mb);
    const bool dead = mn == -INFINITY;  // nothing seen so far (no sink) and nothing visible in this step
    const float p = (dead || s == -INFINITY) ? 0.f : expf(s - mn);
    const float corr = (dead || m == -INFINITY) ? 0.f : expf(m - mn);
    ps[tid] = p;
    const float bs = blk_sum(p, red);  // its barriers also publish ps / pbase
    l = l * corr + bs;
    const int np = min(WA_KEYS / PAGE, walk.count - p0);
#pragma unroll
    for (int a = 0; a < WA_ACC; ++a) {
      const int c = a * 256 + tid;
      if (c < nv) {
        float x = acc[a] * corr;
        for (int pp = 0; pp < np; ++pp) {
          const T* vp = cache + pbase[pp] + (long)PAGE * nk + (long)(c0 + c) * PAGE;
          for (int k = 0; k < PAGE; k += RUN) {
            T v[RUN];
            *reinterpret_cast<u32x4*>(v) = *reinterpret_cast<const u32x4*>(vp + k);
#pragma unroll
            for (int e = 0; e < RUN; ++e) x = fmaf(ps[pp * PAGE + k + e], (float)v[e], x);
          }
        }
        acc[a] = x;
      }
    }
    m = mn;
    __syncthreads();
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int a = 0; a < WA_ACC; ++a) {
    const int c = a * 256 + tid;
    if (c < nv) out[(row * heads + head) * (long)nv + c] = acc[a] * inv;
  }
}

// Matrix-core kernel (bf16; DIM channels per key, VALL = kv_heads * vdim value channels).  A workgroup takes a
// tile of up to 64 query slots = (row, query head of ONE key/value group) pairs of consecutive rows of one
// sequence, so all its slots score against the same keys; wave w owns slots 16 w .. 16 w + 15 end to end
// (queries as B operands, the [16 x VALL] output in registers).  Per visited page the workgroup stages
//   K image   [64 keys][DIM]   (+16 B row padding): A operand of S^T = K Q^T
//   V^T image [VALL][64 keys]  (+16 B row padding): A operand of O^T = V^T P^T   (the page stores V transposed)
// with 16-byte copies.  The rows of a 16-key score tile are taken from the K image in the order that leaves a
// lane with 8 consecutive keys per 32 (v_mfma 16x16x32: lane = slot l % 16, rows 4 (l / 16) + e), so the
// probabilities go from the first product's accumulators into the second without leaving the lane.
// Scores are capped, masked by window / kept first tokens and normalised online in fp32; a sink logit starts
// the running state (max = sink, sum = 1).  The next page's loads are in flight while a page is multiplied.
template <int DIM, int VALL, int NSUB>
__global__ __launch_bounds__(256) void window_mfma_kernel(
    const uint16_t* __restrict__ q, long q_stride, const uint16_t* __restrict__ cache, long page_stride,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ tiles,
    const int* __restrict__ positions, const float* __restrict__ sink, float* __restrict__ out, int heads, int kv_heads,
    int window, int keep_first, float scale, float softcap, int splits, float* __restrict__ ws_o,
    float* __restrict__ ws_ml, int n_chunks, int own, int mode, int pool, long pool_off, int maps) {
  // mode / pool / pool_off: see PageWalk.  maps (own only): key heads per value head
  // own: a slot's weights meet the values of its own KV head only (n_chunks chunks of VALL channels per KV head,
  // out [rows, heads, n_chunks * VALL]); else those of every KV head (n_chunks chunks over all of them)
  constexpr int KS = DIM / 32;
  constexpr int DT = VALL / 16;
  constexpr int PK = DIM * 2 + 16;
  constexpr int PV = PAGE * 2 + 16;
  constexpr int KB = DIM * PAGE / 8 / 256;   // 16-byte chunks of the K tile per thread
  constexpr int VB = VALL * PAGE / 8 / 256;  // and of the V^T tile
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* kimg = lds;
  char* vimg = lds + PAGE * PK;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c16 = lane & 15, g = lane >> 4;
  // value channels beyond VALL are taken in chunks by workgroups of their own (each scores the keys again)
  const int group = blockIdx.y / n_chunks, chunk = blockIdx.y % n_chunks, rep = heads / kv_heads;
  const long vall_total = (long)n_chunks * VALL;
  int seq, row0, n_rows, pos0;
  if (tiles) {
    const int* e = tiles + 4 * blockIdx.x;
    seq = e[0], row0 = e[1], n_rows = e[2], pos0 = e[3];
  } else {  // decode rows: row r is sequence r
    seq = row0 = blockIdx.x, n_rows = 1, pos0 = positions[blockIdx.x];
  }
  if (seq < 0) return;
  // a wave owns NSUB runs of 16 slots: every K and V^T fragment it reads from LDS serves all of them
  const int n_slots = n_rows * rep;
  bool valid[NSUB];
  int head[NSUB], my_pos[NSUB], my_blocks[NSUB];
  long row[NSUB];
#pragma unroll
  for (int u = 0; u < NSUB; ++u) {
    const int slot = (wave * NSUB + u) * 16 + c16;
    valid[u] = slot < n_slots;
    const int tok = valid[u] ? slot / rep : 0;
    head[u] = group * rep + (valid[u] ? slot % rep : 0);
    row[u] = row0 + tok;
    my_pos[u] = valid[u] ? pos0 + tok : -1;
    my_blocks[u] = pool > 0 ? seen_blocks(my_pos[u], window, pool) : 0;
  }
  const bool wave_active = wave * NSUB * 16 < n_slots;  // wave-uniform
  const PageWalk walk(pos0, pos0 + n_rows - 1, window, keep_first, mode, pool);
  const int* bt = block_tables + (long)seq * bt_stride;
  const long k_off = (long)group * DIM, k_row = (long)kv_heads * DIM, v_off = (long)PAGE * kv_heads * DIM;

  bf16x8 qf[NSUB][KS];
  float m[NSUB], l[NSUB];
  f32x4 o[NSUB][DT];
  // key-range splits (decode rows in front of long windows): split blockIdx.z walks its share of the pages and
  // leaves an unnormalised partial (o, max, sum); window_merge_kernel adds the sink and normalises
  const int per = (walk.count + splits - 1) / splits;
  const int i_begin = blockIdx.z * per, i_end = min(walk.count, i_begin + per);
#pragma unroll
  for (int u = 0; u < NSUB; ++u) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (valid[u]) v = *reinterpret_cast<const u32x4*>(q + row[u] * q_stride + (long)head[u] * DIM + 32 * ks + 8 * g);
      qf[u][ks] = __builtin_bit_cast(bf16x8, v);
    }
    const bool seeded = splits == 1 && sink && valid[u];
    m[u] = seeded ? sink[head[u]] : -INFINITY;
    l[u] = seeded ? 1.f : 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[u][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  u32x4 kb[KB], vb[VB];
  auto fetch = [&](int i) {
    const uint16_t* src = cache + (long)bt[walk.page(i)] * page_stride + (walk.pooled(i) ? pool_off : 0);
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      const int id = tid + 256 * b, dc = id % (DIM / 8), key = id / (DIM / 8);
      kb[b] = *reinterpret_cast<const u32x4*>(src + key * k_row + k_off + 8 * dc);
    }
#pragma unroll
    for (int b = 0; b < VB; ++b)
      vb[b] = *reinterpret_cast<const u32x4*>(src + v_off + (long)(own ? group / maps * n_chunks + chunk : chunk) * VALL * PAGE +
                                              (long)(tid + 256 * b) * 8);
  };
  auto stash = [&]() {
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      const int id = tid + 256 * b, dc = id % (DIM / 8), key = id / (DIM / 8);
      *reinterpret_cast<u32x4*>(kimg + key * PK + 16 * dc) = kb[b];
    }
#pragma unroll
    for (int b = 0; b < VB; ++b) {
      const int id = tid + 256 * b;
      *reinterpret_cast<u32x4*>(vimg + (id >> 3) * PV + 16 * (id & 7)) = vb[b];
    }
  };
  // K image row of score-tile row c16 in tile nt: key 32 (nt / 2) + 8 (c16 / 4) + 4 (nt % 2) + c16 % 4
  int krow[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) krow[nt] = (32 * (nt >> 1) + 8 * (c16 >> 2) + 4 * (nt & 1) + (c16 & 3)) * PK + 16 * g;
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;

  if (i_begin < i_end) fetch(i_begin);
  for (int i = i_begin; i < i_end; ++i) {
    __syncthreads();  // the previous page's fragment reads are done
    stash();
    __syncthreads();
    if (i + 1 < i_end) fetch(i + 1);
    if (!wave_active) continue;
    const int j0 = walk.page(i) * PAGE;
    const bool pooled = walk.pooled(i);
    f32x4 s[NSUB][4];
#pragma unroll
    for (int u = 0; u < NSUB; ++u)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) s[u][nt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(kimg + krow[nt] + 64 * ks);
#pragma unroll
        for (int u = 0; u < NSUB; ++u) s[u][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[u][ks], s[u][nt], 0, 0, 0);
      }
    bf16x8 pf[NSUB][2];
    bool rescale = false;
    float corr[NSUB];
#pragma unroll
    for (int u = 0; u < NSUB; ++u) {
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = j0 + 32 * (nt >> 1) + 8 * g + 4 * (nt & 1) + e;
          float v = -INFINITY;
          if (pooled ? j < my_blocks[u] : key_seen(j, my_pos[u], window, keep_first, mode)) {
            v = s[u][nt][e] * scale;
            if (softcap > 0.f) {  // cap * tanh(v / cap), tanh(x) = 1 - 2 / (exp(2 x) + 1)
              const float x = v * inv_cap;
              v = softcap * (1.f - 2.f / (__expf(2.f * x) + 1.f));
            }
          }
          s[u][nt][e] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mn = fmaxf(m[u], mx);
      const bool dead = mn == -INFINITY;
      corr[u] = (dead || m[u] == -INFINITY) ? (dead ? 1.f : 0.f) : __expf(m[u] - mn);
      float psum = 0.f;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float pv = dead ? 0.f : __expf(s[u][nt][e] - mn);
          s[u][nt][e] = pv;
          psum += pv;
        }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l[u] = l[u] * corr[u] + psum;
      m[u] = mn;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        u32x4 w = {pack_bf16x2(s[u][2 * kk][0], s[u][2 * kk][1]), pack_bf16x2(s[u][2 * kk][2], s[u][2 * kk][3]),
                   pack_bf16x2(s[u][2 * kk + 1][0], s[u][2 * kk + 1][1]),
                   pack_bf16x2(s[u][2 * kk + 1][2], s[u][2 * kk + 1][3])};
        pf[u][kk] = __builtin_bit_cast(bf16x8, w);
      }
      rescale = rescale || !__all(corr[u] == 1.f);
    }
    if (rescale) {
#pragma unroll
      for (int u = 0; u < NSUB; ++u)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[u][dt] *= corr[u];
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(vimg + (16 * dt + c16) * PV + 16 * (4 * kk + g));
#pragma unroll
        for (int u = 0; u < NSUB; ++u) o[u][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf[u][kk], o[u][dt], 0, 0, 0);
      }
  }
#pragma unroll
  for (int u = 0; u < NSUB; ++u) {
    if (!valid[u]) continue;
    if (splits == 1) {
      const float inv = l[u] > 0.f ? 1.f / l[u] : 0.f;
      float* dst = out + (row[u] * heads + head[u]) * vall_total + (long)chunk * VALL + 4 * g;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(dst + 16 * dt) = o[u][dt] * inv;
    } else {
      const long rec = (row[u] * heads + head[u]) * splits + blockIdx.z;
      float* dst = ws_o + rec * vall_total + (long)chunk * VALL + 4 * g;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(dst + 16 * dt) = o[u][dt];
      if (g == 0 && chunk == 0) {
        ws_ml[2 * rec] = m[u];
        ws_ml[2 * rec + 1] = l[u];
      }
    }
  }
}

// One workgroup per (row, head): out = sum_s o_s exp(m_s - M) / (sum_s l_s exp(m_s - M) + exp(sink - M))
__global__ __launch_bounds__(128) void window_merge_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                                                           const float* __restrict__ sink, float* __restrict__ out,
                                                           int heads, int vall, int splits) {
  const long pair = blockIdx.x;
  const int head = (int)(pair % heads);
  float big = sink ? sink[head] : -INFINITY;
  for (int s = 0; s < splits; ++s) big = fmaxf(big, ws_ml[2 * (pair * splits + s)]);
  float den = sink ? __expf(sink[head] - big) : 0.f;
  for (int s = 0; s < splits; ++s) {
    const float ms = ws_ml[2 * (pair * splits + s)];
    if (ms != -INFINITY) den += ws_ml[2 * (pair * splits + s) + 1] * __expf(ms - big);
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  for (int c = threadIdx.x; c < vall; c += 128) {
    float acc = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float ms = ws_ml[2 * (pair * splits + s)];
      if (ms != -INFINITY) acc += ws_o[(pair * splits + s) * vall + c] * __expf(ms - big);
    }
    out[pair * vall + c] = acc * inv;
  }
}

// One workgroup per row.  STAGED: KV head by KV head, the weighted values of every query head on that KV head
// (u[:, kv, :], heads x vdim floats) go through LDS in whole float4, since every one of them is read by all the
// heads of the group; else every output reads its inputs from global memory.
template <typename T, bool STAGED>
__global__ __launch_bounds__(256) void mix_heads_kernel(const float* __restrict__ u, const float* __restrict__ talk,
                                                        T* __restrict__ y, int heads, int kv_heads, int vdim) {
  extern __shared__ float us[];
  const long row = blockIdx.x;
  const int rep = heads / kv_heads;
  const float* ur = u + row * (long)heads * kv_heads * vdim;
  T* yr = y + row * (long)heads * vdim;
  if (!STAGED) {
    for (int e = threadIdx.x; e < heads * vdim; e += 256) {
      const int h = e / vdim, c = e - h * vdim;
      const int own = h / rep;
      float acc = 0.f;
      for (int g = 0; g < heads; ++g) acc = fmaf(talk[h * heads + g], ur[((long)g * kv_heads + own) * vdim + c], acc);
      Cv<T>::st(yr + e, acc);
    }
    return;
  }
  const int quads = vdim >> 2;
  for (int own = 0; own < kv_heads; ++own) {
    __syncthreads();
    for (int e = threadIdx.x; e < heads * quads; e += 256) {
      const int g = e / quads, c4 = e - g * quads;
      *reinterpret_cast<f32x4*>(us + g * vdim + 4 * c4) =
          *reinterpret_cast<const f32x4*>(ur + ((long)g * kv_heads + own) * vdim + 4 * c4);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < rep * vdim; e += 256) {
      const int h = own * rep + e / vdim, c = e % vdim;
      float acc = 0.f;
      for (int g = 0; g < heads; ++g) acc = fmaf(talk[h * heads + g], us[g * vdim + c], acc);
      Cv<T>::st(yr + (long)h * vdim + c, acc);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void xielu_kernel(const T* __restrict__ x, T* __restrict__ y, long n,
                                                    const float* __restrict__ act) {
  const float ap = act[0], an = act[1];
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const float z = Cv<T>::ld(x + i);
    const float v = z > 0.f ? fmaf(ap * z, z, 0.5f * z) : fmaf(an, expm1f(z) - z, 0.5f * z);
    Cv<T>::st(y + i, v);
  }
}

}  // namespace

#define SM_DISPATCH(dt, CALL)                         \
  if ((dt) == 0) { using T = bf16_t; CALL; }          \
  else if ((dt) == 1) { using T = float; CALL; }      \
  else return 1;

VPSA_EXPORT int vpsa_add_dyt(float* residual, const void* d1, long s1, float c1, const void* d2, long s2, float c2,
                             const float* w, const float* b, const float* alpha, void* y, int rows, int n, int dt,
                             hipStream_t stream) {
  if (rows <= 0) return 0;
  SM_DISPATCH(dt, (add_dyt_kernel<T><<<rows, 256, 0, stream>>>(residual, (const T*)d1, s1, c1, (const T*)d2, s2, c2, w, b,
                                                               alpha, (T*)y, n)));
  return 0;
}

// Rows of the state a lane holds and lanes per column group for a head of `dim` rows.  16 rows x 4 columns is the
// largest tile that still leaves six waves per SIMD (128 x 256 states, 8192 rows: 1.25 ms against 2.3 ms with 32
// rows and 1.4 ms with 8, which pays in cross-lane sums); heads beyond 1024 rows are refused.
static void scan_shape(int dim, int* rpt, int* r) {
  static const int forced = getenv("VPSA_SCAN_ROWS") ? atoi(getenv("VPSA_SCAN_ROWS")) : 0;  // A/B runs: 8, 16 or 32
  int p = (forced == 8 || forced == 16 || forced == 32) ? forced : (dim <= 32 ? 8 : 16);
  int lanes = 1;
  while (lanes * p < dim) lanes <<= 1;
  *rpt = p;
  *r = lanes;
}

// pieces: nullptr = every sequence in one go (its rows from seq_cu); else int32 [n_pieces][3] = (sequence, first row,
// rows) in sequence order, seq_pieces int32 [n_seqs + 1] = a sequence's first piece, and the workspaces
// ws_state fp32 [n_pieces, heads, dim, vdim], ws_decay fp32 [n_pieces, heads, dim].  prep: fp32 workspace
// [rows, heads, 2 (3 when gated), dim].  fold: every decay's 16th power is well inside fp32's range (the kernel
// then folds the decay into the staged keys and queries).
// prepared: `prep` already holds q' | k' | a for every row (the caller's own gates): nothing is prepared here, the
// pieces' decays come from it, and `proj` only serves the values (vsrc columns per head; with unit_col the state has
// one more column, fed with ones).
static int scan_run(const void* proj, long p_stride, int q_col, int k_col, int v_col, int heads, int dim, int vdim,
                    float* state, long state_stride, const int* seq_cu, const int* seq_state, int n_seqs,
                    const int* positions, const float* decay, const float* cos_sin, int rot_dims, int layout,
                    float k_scale, const float* gate_bias, const float* gate_lower, float* out, int gated,
                    const int* pieces, const int* seq_pieces, int n_pieces, float* ws_state, float* ws_decay,
                    float* prep, int rows, int fold, int dt, hipStream_t stream, int prepared, int vsrc, int unit_col,
                    int act = 0) {
  // act: 1 = q, k and v pass through silu (fixed-decay form)
  if (act && (gated || prepared || rot_dims)) return 6;
  if (n_seqs <= 0 || rows <= 0) return 0;
  int rpt, r;
  scan_shape(dim, &rpt, &r);
  if (r > 64) return 2;
  const int dimp = r * rpt, cols = (256 / r) * 4;
  const int per_tok = (gated ? 3 : 2) * dimp + cols;
  int tb = (48 * 1024 / 4) / per_tok;
  if (tb > 16) tb = 16;
  if (tb < 1) return 3;
  const size_t lds = (size_t)tb * per_tok * sizeof(float);
  const int col_blocks = (vdim + cols - 1) / cols;
#define SCAN(RPT, G, F, PH, NZ)                                                                                        \
  recurrent_scan_kernel<T, RPT, G, F, PH><<<dim3(col_blocks, heads, NZ), 256, lds, stream>>>(                          \
      (const T*)proj, p_stride, v_col, heads, dim, vdim, prep, state, state_stride, seq_cu, seq_state, positions,     \
      decay, out, r, tb, pieces, ws_state, vsrc, unit_col, act)
#define SCAN_R(G, F, PH, NZ)                       \
  if (rpt == 8) SCAN(8, G, F, PH, NZ);             \
  else if (rpt == 16) SCAN(16, G, F, PH, NZ);      \
  else SCAN(32, G, F, PH, NZ);
#define SCAN_G(PH, NZ)                             \
  if (gated) { SCAN_R(true, false, PH, NZ) }       \
  else if (fold) { SCAN_R(false, true, PH, NZ) }   \
  else { SCAN_R(false, false, PH, NZ) }
  if (prepared) {
  } else if (gated) {
    SM_DISPATCH(dt, (scan_prepare_kernel<T, true><<<rows, 256, 0, stream>>>((const T*)proj, p_stride, q_col, k_col, heads,
                                                                            dim, positions, cos_sin, rot_dims, layout,
                                                                            k_scale, gate_bias, gate_lower, prep, act)));
  } else {
    SM_DISPATCH(dt, (scan_prepare_kernel<T, false><<<rows, 256, 0, stream>>>((const T*)proj, p_stride, q_col, k_col, heads,
                                                                             dim, positions, cos_sin, rot_dims, layout,
                                                                             k_scale, gate_bias, gate_lower, prep, act)));
  }
  if (!pieces) {
    SM_DISPATCH(dt, SCAN_G(0, n_seqs));
    return 0;
  }
  if (n_pieces <= 0 || !seq_pieces || !ws_state || !ws_decay) return 4;
  if (prepared) {
    scan_decay_prep_kernel<<<dim3(n_pieces, heads), 128, 0, stream>>>(prep, heads, dim, pieces, ws_decay);
  } else if (gated) {
    SM_DISPATCH(dt, (scan_decay_kernel<T, true><<<dim3(n_pieces, heads), 128, 0, stream>>>(
                        (const T*)proj, p_stride, k_col, heads, dim, decay, gate_bias, gate_lower, pieces, ws_decay)));
  } else {
    SM_DISPATCH(dt, (scan_decay_kernel<T, false><<<dim3(n_pieces, heads), 128, 0, stream>>>(
                        (const T*)proj, p_stride, k_col, heads, dim, decay, gate_bias, gate_lower, pieces, ws_decay)));
  }
  SM_DISPATCH(dt, SCAN_G(1, n_pieces));
  scan_propagate_kernel<<<dim3((dim * vdim + 255) / 256, heads, n_seqs), 256, 0, stream>>>(
      ws_state, ws_decay, state, state_stride, seq_cu, seq_state, seq_pieces, positions, heads, dim, vdim);
  SM_DISPATCH(dt, SCAN_G(2, n_pieces));
#undef SCAN
#undef SCAN_R
#undef SCAN_G
  return 0;
}

VPSA_EXPORT int vpsa_recurrent_scan(const void* proj, long p_stride, int q_col, int k_col, int v_col, int heads, int dim,
                                    int vdim, float* state, long state_stride, const int* seq_cu, const int* seq_state,
                                    int n_seqs, const int* positions, const float* decay, const float* cos_sin,
                                    int rot_dims, int layout, float k_scale, const float* gate_bias,
                                    const float* gate_lower, float* out, int gated, const int* pieces,
                                    const int* seq_pieces, int n_pieces, float* ws_state, float* ws_decay, float* prep,
                                    int rows, int fold, int act, int dt, hipStream_t stream) {
  return scan_run(proj, p_stride, q_col, k_col, v_col, heads, dim, vdim, state, state_stride, seq_cu, seq_state, n_seqs,
                  positions, decay, cos_sin, rot_dims, layout, k_scale, gate_bias, gate_lower, out, gated, pieces,
                  seq_pieces, n_pieces, ws_state, ws_decay, prep, rows, fold, dt, stream, 0, vdim, 0, act);
}

// The recurrence over rows the caller prepared: prep fp32 [rows, heads, 3, dim] = q' | k' | a, values from `v`
// (row stride v_stride, heads side by side from column v_col, vsrc columns each).  The state has vdim columns per
// key channel: vsrc, or with unit_col at least vsrc + 1 (column vsrc accumulates k' alone: read out by q' it is the
// normaliser's dot product).  out fp32 [rows, heads, vdim].
VPSA_EXPORT int vpsa_prepared_scan(const void* v, long v_stride, int v_col, int vsrc, int unit_col, int heads, int dim,
                                   int vdim, float* prep, float* state, long state_stride, const int* seq_cu,
                                   const int* seq_state, int n_seqs, const int* positions, float* out,
                                   const int* pieces, const int* seq_pieces, int n_pieces, float* ws_state,
                                   float* ws_decay, int rows, int dt, hipStream_t stream) {
  if (vsrc + (unit_col ? 1 : 0) > vdim) return 5;
  return scan_run(v, v_stride, 0, 0, v_col, heads, dim, vdim, state, state_stride, seq_cu, seq_state, n_seqs, positions,
                  nullptr, nullptr, 0, 0, 1.f, nullptr, nullptr, out, 1, pieces, seq_pieces, n_pieces, ws_state,
                  ws_decay, prep, rows, 0, dt, stream, 1, vsrc, unit_col);
}

VPSA_EXPORT int vpsa_gla_prepare(const void* proj, long p_stride, int q_col, int k_col, const void* z, long z_stride,
                                 const float* z_bias, int heads, int dim, float q_scale, float tau, float* prep,
                                 int rows, int dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  SM_DISPATCH(dt, (gla_prepare_kernel<T><<<rows, 256, 0, stream>>>((const T*)proj, p_stride, q_col, k_col, (const T*)z,
                                                                   z_stride, z_bias, heads, dim, q_scale, 1.f / tau, prep)));
  return 0;
}

// logits fp32 [rows, 2 heads] = input-gate | forget-gate pre-activations (without their biases); m_state: the
// running maxima's place in the state pool (heads floats per slot).  Leaves prep (q * q_scale | k * write | decay)
// and mrow fp32 [rows, heads] (the running maximum after every token); ab fp32 [rows, heads, 2] is workspace.
VPSA_EXPORT int vpsa_mlstm_prepare(const void* proj, long p_stride, int q_col, int k_col, const float* logits,
                                   const float* bias_i, const float* bias_f, float cap, int heads, int dim,
                                   float q_scale, float* m_state, long state_stride, const int* seq_cu,
                                   const int* seq_state, int n_seqs, const int* positions, float* ab, float* mrow,
                                   float* prep, int rows, int dt, hipStream_t stream) {
  if (rows <= 0 || n_seqs <= 0) return 0;
  mlstm_gates_kernel<<<dim3(n_seqs, heads), 64, 0, stream>>>(logits, bias_i, bias_f, cap, heads, m_state, state_stride,
                                                            seq_cu, seq_state, positions, ab, mrow);
  SM_DISPATCH(dt, (mlstm_prepare_kernel<T><<<rows, 256, 0, stream>>>((const T*)proj, p_stride, q_col, k_col, ab, heads,
                                                                     dim, q_scale, prep)));
  return 0;
}

VPSA_EXPORT int vpsa_head_finish(const float* o, int ostride, const float* stab, int unit, const float* w, int w_heads,
                                 const void* gate, long g_stride, int gate_act, void* y, int rows, int heads, int vdim,
                                 float eps, int dt, hipStream_t stream) {
  const long pairs = (long)rows * heads;
  if (pairs <= 0) return 0;
  if (ostride < vdim + (stab ? 1 : 0)) return 2;
  if (vdim >= 1024) {
    SM_DISPATCH(dt, (head_rms_wide_kernel<T><<<(unsigned)pairs, 256, 0, stream>>>(
                        o, ostride, stab, unit, w, w_heads, (const T*)gate, g_stride, gate_act, (T*)y, heads, vdim, eps)));
    return 0;
  }
  SM_DISPATCH(dt, (head_rms_kernel<T><<<(unsigned)((pairs + 3) / 4), 256, 0, stream>>>(
                      o, ostride, stab, unit, w, w_heads, (const T*)gate, g_stride, gate_act, (T*)y, pairs, heads, vdim,
                      eps)));
  return 0;
}

VPSA_EXPORT int vpsa_head_rms(const float* o, const float* w, const void* gate, long g_stride, void* y, int rows,
                              int heads, int vdim, float eps, int dt, hipStream_t stream) {
  return vpsa_head_finish(o, vdim, nullptr, 1, w, 0, gate, g_stride, 0, y, rows, heads, vdim, eps, dt, stream);
}

// proj rows: q | k | v when own (the layer caches its keys and values), q alone otherwise.
VPSA_EXPORT int vpsa_qk_norm_write(const void* proj, long p_stride, int heads, int kv_heads, int dim, int vdim, int own,
                                   const int* positions, const long* slots, float eps, float coef, float every,
                                   void* q_out, void* cache, long page_stride, int rows, int v_heads, const float* qw,
                                   const float* kw, const float* cos_sin, int rot_dims, int layout, int dt,
                                   hipStream_t stream) {
  if (rows <= 0) return 0;
  if (coef != 0.f && !(every > 0.f)) return 2;
  if (rot_dims < 0 || rot_dims > dim || rot_dims % 2 || (rot_dims && !cos_sin) || v_heads < 1) return 3;
  const int head_runs = rows <= 512 ? (heads + (own ? kv_heads : 0) + 3) / 4 : 1;
  SM_DISPATCH(dt, (qk_norm_write_kernel<T><<<dim3(rows, head_runs), 256, 0, stream>>>(
                      (const T*)proj, p_stride, heads, kv_heads, dim, vdim, own, positions, slots, eps, coef, every,
                      (T*)q_out, (T*)cache, page_stride, v_heads, qw, kw, rot_dims ? cos_sin : nullptr, rot_dims, layout)));
  return 0;
}

// nk / nv: key and value channels per token of the layer's page regions (all heads)
VPSA_EXPORT int vpsa_pool_blocks(void* cache, long page_stride, long pool_off, const int* block_tables, int bt_stride,
                                 const int* row_seq, const int* positions, const long* slots, int rows, int nk, int nv,
                                 int pool, int dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (pool < 1 || pool_off < (long)PAGE * (nk + nv)) return 2;
  SM_DISPATCH(dt, (pool_blocks_kernel<T><<<dim3((rows + POOL_ROWS - 1) / POOL_ROWS, (nk + nv + 255) / 256), 256, 0, stream>>>(
                      (T*)cache, page_stride, pool_off, block_tables, bt_stride, row_seq, positions, slots, rows, nk, nv,
                      pool)));
  return 0;
}

VPSA_EXPORT int vpsa_diff_heads(const float* u, void* y, int rows, int heads, int kv_heads, int vdim, float lambda,
                                float eps, float post, int dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (kv_heads < 1 || heads % kv_heads) return 2;
  const long pairs = (long)rows * heads;
  SM_DISPATCH(dt, (diff_heads_kernel<T><<<(unsigned)((pairs + 3) / 4), 256, 0, stream>>>(
                      u, (T*)y, pairs, heads, heads / kv_heads, vdim, lambda, eps, post)));
  return 0;
}

VPSA_EXPORT int vpsa_short_conv_qkv(const void* proj, long p_stride, const float* conv_w, int taps, int heads,
                                    int kv_heads, int dim, int vdim, float* state, long state_stride,
                                    const int* row_seq, const int* seq_cu, const int* seq_state, int n_seqs,
                                    const int* positions, const long* slots, const float* cos_sin, int rot_dims,
                                    int layout, void* q_out, void* cache, long page_stride, int rows, int dt,
                                    hipStream_t stream) {
  if (rows <= 0) return 0;
  const int chans = heads * dim + kv_heads * (dim + vdim);
  if ((size_t)chans * 4 > 60 * 1024 || taps < 1) return 2;
  SM_DISPATCH(dt, (short_conv_qkv_kernel<T><<<rows, 256, (size_t)chans * 4, stream>>>(
                      (const T*)proj, p_stride, conv_w, taps, heads, kv_heads, dim, vdim, state, state_stride, row_seq,
                      seq_cu, seq_state, positions, slots, cos_sin, rot_dims, layout, (T*)q_out, (T*)cache, page_stride)));
  if (taps > 1) {
    SM_DISPATCH(dt, (conv_tail_kernel<T><<<n_seqs, 256, 0, stream>>>((const T*)proj, p_stride, taps, chans, state,
                                                                     state_stride, seq_cu, seq_state, positions)));
  }
  return 0;
}

VPSA_EXPORT int vpsa_window_attention(const void* q, long q_stride, const void* cache, long page_stride,
                                      const int* block_tables, int bt_stride, const int* row_seq, const int* positions,
                                      const float* sink, float* out, int rows, int heads, int kv_heads, int dim, int vdim,
                                      int window, int keep_first, float scale, float softcap, int own, int mode,
                                      int pool, long pool_off, int maps, int dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if ((own ? vdim : kv_heads * vdim) > 256 * WA_ACC || (size_t)dim * 4 > 32 * 1024 || heads % kv_heads) return 2;
  if (window < 1 || maps < 1 || kv_heads % maps || (maps > 1 && !own) || (pool > 0 && (keep_first || mode))) return 4;
  dim3 grid(rows, heads);
  SM_DISPATCH(dt, (window_attention_kernel<T><<<grid, 256, (size_t)dim * 4, stream>>>(
                      (const T*)q, q_stride, (const T*)cache, page_stride, block_tables, bt_stride, row_seq, positions,
                      sink, out, heads, kv_heads, dim, vdim, window, keep_first, scale, softcap, own, mode, pool, pool_off,
                      maps)));
  return 0;
}

// Value channels a workgroup of the matrix-core kernel takes (0: the shape is not tiled).
static int window_chunk(int vall) {
  for (int c = 512; c >= 128; c >>= 1)
    if (vall % c == 0) return c;
  return 0;
}

VPSA_EXPORT int vpsa_window_mfma_supported(int heads, int kv_heads, int dim, int vdim, int own) {
  return (dim == 64 || dim == 128) && window_chunk(own ? vdim : kv_heads * vdim) > 0 && heads % kv_heads == 0 &&
         heads / kv_heads <= 64;
}

// Runs of 16 slots per wave in prefill tiles.  Two (a tile of 128 slots, every LDS fragment read half as often per
// slot) need 256 accumulator registers per lane at 512 value channels; the compiler keeps them in the 256 arch
// registers and spills (1.4 ms against 0.6 ms per 8192 rows), so one it is until the accumulators are placed by hand.
#define WINDOW_PREFILL_SUB 1

template <int DIM, int VALL, int NSUB>
static int launch_window_mfma(const void* q, long q_stride, const void* cache, long page_stride, const int* block_tables,
                              int bt_stride, const int* tiles, const int* positions, const float* sink, float* out,
                              int n_tiles, int heads, int kv_heads, int window, int keep_first, float scale,
                              float softcap, int splits, float* ws_o, float* ws_ml, int n_chunks, int own, int mode,
                              int pool, long pool_off, int maps, hipStream_t st) {
  constexpr int LDS = PAGE * (DIM * 2 + 16) + VALL * (PAGE * 2 + 16);
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)window_mfma_kernel<DIM, VALL, NSUB>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            LDS) != hipSuccess)
      return -2;
    attr_set = true;
  }
  window_mfma_kernel<DIM, VALL, NSUB><<<dim3(n_tiles, kv_heads * n_chunks, splits), dim3(256), LDS, st>>>(
      (const uint16_t*)q, q_stride, (const uint16_t*)cache, page_stride, block_tables, bt_stride, tiles, positions, sink,
      out, heads, kv_heads, window, keep_first, scale, softcap, splits, ws_o, ws_ml, n_chunks, own, mode, pool, pool_off,
      maps);
  if (splits > 1)  // decode rows only: row r of the launch is row r of out
    window_merge_kernel<<<n_tiles * heads, 128, 0, st>>>(ws_o, ws_ml, sink, out, heads, VALL * n_chunks, splits);
  return 0;
}

// (row, query head) pairs of one prefill tile of the matrix-core kernel
VPSA_EXPORT int vpsa_window_tile_slots() { return 64 * WINDOW_PREFILL_SUB; }

// tiles: int32 [n_tiles][4] = (sequence, first row, rows, position of the first row), -1 sequence = skip;
// nullptr: n_tiles decode rows, row r = sequence r at positions[r].
VPSA_EXPORT int vpsa_window_attention_mfma(const void* q, long q_stride, const void* cache, long page_stride,
                                           const int* block_tables, int bt_stride, const int* tiles,
                                           const int* positions, const float* sink, float* out, int n_tiles, int heads,
                                           int kv_heads, int dim, int vdim, int window, int keep_first, float scale,
                                           float softcap, int splits, float* ws_o, float* ws_ml, int own, int mode,
                                           int pool, long pool_off, int maps, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (window < 1 || maps < 1 || kv_heads % maps || (maps > 1 && !own) || (pool > 0 && (keep_first || mode))) return 4;
  if (!vpsa_window_mfma_supported(heads, kv_heads, dim, vdim, own)) return 2;
  if (splits < 1 || (splits > 1 && (tiles || !ws_o || !ws_ml))) return 3;  // splits are for decode rows
  const int vall = window_chunk(own ? vdim : kv_heads * vdim), n_chunks = (own ? vdim : kv_heads * vdim) / vall;
#define WM(D, V)                                                                                                      \
  if (dim == D && vall == V) {                                                                                        \
    if (tiles)                                                                                                        \
      return launch_window_mfma<D, V, WINDOW_PREFILL_SUB>(q, q_stride, cache, page_stride, block_tables, bt_stride,    \
                                                          tiles, positions, sink, out, n_tiles, heads, kv_heads,      \
                                                          window, keep_first, scale, softcap, splits, ws_o, ws_ml,     \
                                                          n_chunks, own, mode, pool, pool_off, maps, stream);         \
    return launch_window_mfma<D, V, 1>(q, q_stride, cache, page_stride, block_tables, bt_stride, tiles, positions,     \
                                       sink, out, n_tiles, heads, kv_heads, window, keep_first, scale, softcap,       \
                                       splits, ws_o, ws_ml, n_chunks, own, mode, pool, pool_off, maps, stream);       \
  }
  WM(64, 128) WM(64, 256) WM(64, 512) WM(128, 128) WM(128, 256) WM(128, 512)
#undef WM
  return 2;
}

VPSA_EXPORT int vpsa_mix_heads(const float* u, const float* talk, void* y, int rows, int heads, int kv_heads, int vdim,
                               int dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  const size_t bytes = (size_t)heads * vdim * 4;
  if (bytes <= 48 * 1024 && vdim % 4 == 0 && ((uintptr_t)u & 15) == 0) {
    SM_DISPATCH(dt, (mix_heads_kernel<T, true><<<rows, 256, bytes, stream>>>(u, talk, (T*)y, heads, kv_heads, vdim)));
  } else {
    SM_DISPATCH(dt, (mix_heads_kernel<T, false><<<rows, 256, 0, stream>>>(u, talk, (T*)y, heads, kv_heads, vdim)));
  }
  return 0;
}

VPSA_EXPORT int vpsa_xielu(const void* x, void* y, long n, const float* act, int dt, hipStream_t stream) {
  if (n <= 0) return 0;
  long blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  SM_DISPATCH(dt, (xielu_kernel<T><<<(unsigned)blocks, 256, 0, stream>>>((const T*)x, (T*)y, n, act)));
  return 0;
}
