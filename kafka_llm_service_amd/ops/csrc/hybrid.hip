// Kernels of the hybrid decoder family (latent attention + Mamba-2 layers, layer norms before and after every
// sublayer, token shift, per-layer token input, depth average) for gfx950.
//
// Every kernel is built for bf16 and for fp32 activations (template AT); the residual stream, the recurrent state,
// every norm's statistics, softmax, rotary products and the recurrence's gates are fp32 in both. Sizes are run-time
// values with no alignment assumptions (channel counts, head sizes and ranks come from the model's config), so rows
// are walked with scalar, lane-consecutive (coalesced) accesses.
//
// A step's rows are described by segments: seg[r] = (first row, rows, first position, state slot), one per sequence
// in the step, and tok_seg[t] = the segment of row t. A segment whose first position is 0 has zero state: its slot is
// written, never read, so reused slots need no clearing.
//
//   ln_shift        layer norm (weight + bias) of the fp32 stream -> AT; with a shift vector each row is moved towards
//                   the previous row's normed value (the slot's state for a segment's first row) - the previous row
//                   is re-normed by the same workgroup, nothing is exchanged between workgroups
//   add_ln          x += layer_norm(y) and, in the same pass over the row, the next sublayer's pre-norm of the new x
//   side_dwa        x += unit_rms(y) * w, push x on the depth stack, x = sum_j a_j stack_j
//   latent_prep     RMS norm of the latent + rotary on the shared key part -> paged cache row; rotary on the query parts
//   latent_attn     all heads of a row against the row's cached [latent | rotary key] rows: one wave per (row, 4
//                   heads), the 64 lanes across the row's dimensions, online softmax, the value pass reusing the key
//                   registers (the values ARE the latent part of the key row)
//   short_conv      causal short convolution (optional bias, silu, residual) with a per-slot tail of raw inputs
//   ssm_scan        the state-space recurrence, one workgroup per (segment, head, column slice), an 8 x 4 state block
//                   per thread in registers, B / C / x / dt of the next tokens staged through LDS, double buffered
//   gated_norm      y * silu(z), RMS norm in groups, weight
#include "common.h"

namespace kafka {
namespace hy {

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)(*p); }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float inv_sqrt(float v) { return 1.0f / sqrtf(v); }

constexpr int NT = 256;

// Workgroup barrier for LDS hand-overs that leaves global loads in flight: __syncthreads() drains vmcnt as well,
// which would stall on every prefetch issued before it. This wave's LDS reads and writes are complete (lgkmcnt 0)
// before it arrives.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// mean and 1 / sqrt(var + eps) of an fp32 or AT row
template <typename XT>
__device__ __forceinline__ void row_stats(const XT* __restrict__ r, int d, float eps, float* red, float& mean,
                                          float& rstd) {
  float s = 0.f;
  for (int i = threadIdx.x; i < d; i += NT) s += ldf(r + i);
  mean = block_sum<NT>(s, red) / (float)d;
  float v = 0.f;
  for (int i = threadIdx.x; i < d; i += NT) {
    const float c = ldf(r + i) - mean;
    v += c * c;
  }
  rstd = inv_sqrt(block_sum<NT>(v, red) / (float)d + eps);
}

template <typename AT>
__global__ __launch_bounds__(NT) void ln_shift_kernel(const float* __restrict__ x, int64_t xs, const AT* __restrict__ w,
                                                      const AT* __restrict__ b, float eps, AT* __restrict__ out,
                                                      int64_t os, int d, const AT* __restrict__ mu,
                                                      const int* __restrict__ tok_seg, const int* __restrict__ seg,
                                                      const float* __restrict__ state, float* __restrict__ last) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const float* xr = x + t * xs;
  float mean, rstd;
  row_stats(xr, d, eps, red, mean, rstd);
  if (mu == nullptr) {
    for (int i = threadIdx.x; i < d; i += NT) stf(out + t * os + i, (xr[i] - mean) * rstd * ldf(w + i) + ldf(b + i));
    return;
  }
  const int sg = tok_seg[t];
  const int q0 = seg[4 * sg], n = seg[4 * sg + 1], p0 = seg[4 * sg + 2], slot = seg[4 * sg + 3];
  const bool first = (t == q0), is_last = (t == q0 + n - 1);
  float mean2 = 0.f, rstd2 = 0.f;
  const float* xp = xr - xs;
  if (!first) row_stats(xp, d, eps, red, mean2, rstd2);  // (uniform per workgroup)
  for (int i = threadIdx.x; i < d; i += NT) {
    const float wi = ldf(w + i), bi = ldf(b + i);
    const float h = (xr[i] - mean) * rstd * wi + bi;
    float prev;
    if (first)
      prev = p0 > 0 ? state[(int64_t)slot * d + i] : 0.f;
    else
      prev = (xp[i] - mean2) * rstd2 * wi + bi;
    stf(out + t * os + i, h + (prev - h) * ldf(mu + i));
    if (is_last) last[(int64_t)sg * d + i] = h;
  }
}

__global__ void scatter_rows_kernel(float* __restrict__ dst, const int* __restrict__ seg, const float* __restrict__ src,
                                    int d) {
  const int r = blockIdx.x;
  const int slot = seg[4 * r + 3];
  for (int i = threadIdx.x; i < d; i += blockDim.x) dst[(int64_t)slot * d + i] = src[(int64_t)r * d + i];
}

// x += ln(y; w, b); MODE 1: out2 = ln(x_new; w2, b2); MODE 2: out2 = x_new (cast)
template <typename AT, int MODE>
__global__ __launch_bounds__(NT) void add_ln_kernel(float* __restrict__ x, int64_t xs, const AT* __restrict__ y,
                                                    int64_t ys, const AT* __restrict__ w, const AT* __restrict__ b,
                                                    float eps, int d, AT* __restrict__ out2, int64_t os,
                                                    const AT* __restrict__ w2, const AT* __restrict__ b2) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const AT* yr = y + t * ys;
  float* xr = x + t * xs;
  float mean, rstd;
  row_stats(yr, d, eps, red, mean, rstd);
  for (int i = threadIdx.x; i < d; i += NT) {
    const float v = xr[i] + ((ldf(yr + i) - mean) * rstd * ldf(w + i) + ldf(b + i));
    xr[i] = v;  // re-read below by the same thread only
    if constexpr (MODE == 2) stf(out2 + t * os + i, v);
  }
  if constexpr (MODE == 1) {
    float m2, r2;
    row_stats(xr, d, eps, red, m2, r2);
    for (int i = threadIdx.x; i < d; i += NT)
      stf(out2 + t * os + i, (xr[i] - m2) * r2 * ldf(w2 + i) + ldf(b2 + i));
  }
}

// ---- the same three row kernels with the row held in registers (d <= NV * 256) -------------------------------------
// A step of few rows (a decode step) has few workgroups, so these kernels are latency-bound: every pass over a row
// that goes back to memory is a dependent round trip. Here each row is loaded once (all its loads in flight together,
// the previous row's and the second operand's too) and the statistics, the second norm and the outputs come from
// registers. The sums run over the same elements in the same order as in the generic kernels above.
template <int NV>
__device__ __forceinline__ void reg_stats(const float (&v)[NV], int d, float eps, float* red, float& mean, float& rstd) {
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k)
    if ((int)threadIdx.x + k * NT < d) s += v[k];
  mean = block_sum<NT>(s, red) / (float)d;
  float q = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k)
    if ((int)threadIdx.x + k * NT < d) {
      const float c = v[k] - mean;
      q += c * c;
    }
  rstd = inv_sqrt(block_sum<NT>(q, red) / (float)d + eps);
}

template <typename AT, int NV>
__global__ __launch_bounds__(NT) void ln_shift_reg_kernel(const float* __restrict__ x, int64_t xs,
                                                          const AT* __restrict__ w, const AT* __restrict__ b, float eps,
                                                          AT* __restrict__ out, int64_t os, int d,
                                                          const AT* __restrict__ mu, const int* __restrict__ tok_seg,
                                                          const int* __restrict__ seg, const float* __restrict__ state,
                                                          float* __restrict__ last) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const float* xr = x + t * xs;
  bool first = true, is_last = false;
  int sg = 0, p0 = 0, slot = 0;
  if (mu != nullptr) {
    sg = tok_seg[t];
    const int q0 = seg[4 * sg], n = seg[4 * sg + 1];
    p0 = seg[4 * sg + 2];
    slot = seg[4 * sg + 3];
    first = (t == q0);
    is_last = (t == q0 + n - 1);
  }
  float v[NV], pv[NV], wv[NV], bv[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int i = threadIdx.x + k * NT;
    const bool in = i < d;
    v[k] = in ? xr[i] : 0.f;
    wv[k] = in ? ldf(w + i) : 0.f;
    bv[k] = in ? ldf(b + i) : 0.f;
    pv[k] = 0.f;
    if (mu != nullptr && in) pv[k] = first ? (p0 > 0 ? state[(int64_t)slot * d + i] : 0.f) : xr[i - xs];
  }
  float mean, rstd, mean2 = 0.f, rstd2 = 0.f;
  reg_stats<NV>(v, d, eps, red, mean, rstd);
  if (mu != nullptr && !first) reg_stats<NV>(pv, d, eps, red, mean2, rstd2);  // (uniform per workgroup)
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int i = threadIdx.x + k * NT;
    if (i < d) {
      const float h = (v[k] - mean) * rstd * wv[k] + bv[k];
      if (mu == nullptr) {
        stf(out + t * os + i, h);
      } else {
        const float prev = first ? pv[k] : (pv[k] - mean2) * rstd2 * wv[k] + bv[k];
        stf(out + t * os + i, h + (prev - h) * ldf(mu + i));
        if (is_last) last[(int64_t)sg * d + i] = h;
      }
    }
  }
}

template <typename AT, int NV, int MODE>
__global__ __launch_bounds__(NT) void add_ln_reg_kernel(float* __restrict__ x, int64_t xs, const AT* __restrict__ y,
                                                        int64_t ys, const AT* __restrict__ w,
                                                        const AT* __restrict__ b, float eps, int d,
                                                        AT* __restrict__ out2, int64_t os, const AT* __restrict__ w2,
                                                        const AT* __restrict__ b2) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  float yv[NV], xv[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int i = threadIdx.x + k * NT;
    yv[k] = i < d ? ldf(y + t * ys + i) : 0.f;
    xv[k] = i < d ? x[t * xs + i] : 0.f;
  }
  float mean, rstd;
  reg_stats<NV>(yv, d, eps, red, mean, rstd);
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int i = threadIdx.x + k * NT;
    if (i < d) {
      xv[k] = xv[k] + ((yv[k] - mean) * rstd * ldf(w + i) + ldf(b + i));
      x[t * xs + i] = xv[k];
      if constexpr (MODE == 2) stf(out2 + t * os + i, xv[k]);
    }
  }
  if constexpr (MODE == 1) {
    float m2, r2;
    reg_stats<NV>(xv, d, eps, red, m2, r2);
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = threadIdx.x + k * NT;
      if (i < d) stf(out2 + t * os + i, (xv[k] - m2) * r2 * ldf(w2 + i) + ldf(b2 + i));
    }
  }
}

template <typename AT, int NV>
__global__ __launch_bounds__(NT) void side_dwa_reg_kernel(float* __restrict__ x, const AT* __restrict__ y, int64_t ys,
                                                          const AT* __restrict__ sw, float eps,
                                                          float* __restrict__ stack, int layer,
                                                          const float* __restrict__ dwa, int64_t T, int d) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int64_t plane = T * d;
  float xv[NV], yv[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int i = threadIdx.x + k * NT;
    xv[k] = i < d ? x[t * d + i] : 0.f;
    yv[k] = (y != nullptr && i < d) ? ldf(y + t * ys + i) : 0.f;
  }
  if (y != nullptr) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) s += yv[k] * yv[k];  // (zeros beyond d)
    const float r = inv_sqrt(block_sum<NT>(s, red) / (float)d + eps);
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = threadIdx.x + k * NT;
      if (i < d) xv[k] += yv[k] * r * ldf(sw + i);
    }
  }
  if (stack != nullptr) {
    float a[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = threadIdx.x + k * NT;
      if (i < d) stack[(int64_t)(layer + 1) * plane + t * d + i] = xv[k];
      a[k] = 0.f;
    }
    if (dwa != nullptr) {
      for (int j = 0; j <= layer; ++j) {  // one plane per turn, the row's NV loads of it in flight together
        const float c = dwa[j];
        const float* pj = stack + (int64_t)j * plane + t * d;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
          const int i = threadIdx.x + k * NT;
          if (i < d) a[k] += c * pj[i];
        }
      }
      const float c = dwa[layer + 1];
#pragma unroll
      for (int k = 0; k < NV; ++k) xv[k] = a[k] + c * xv[k];
    }
  }
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int i = threadIdx.x + k * NT;
    if (i < d) x[t * d + i] = xv[k];
  }
}

template <typename AT>
__global__ void gelu_mul_kernel(const AT* __restrict__ gu, int64_t gs, AT* __restrict__ out, int64_t T, int F) {
  const int64_t n = T * F;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / F;
    const int f = (int)(i - t * F);
    stf(out + i, gelu_tanh(ldf(gu + t * gs + f)) * ldf(gu + t * gs + F + f));
  }
}

template <typename AT>
__global__ void side_gate_kernel(const AT* __restrict__ sg, int64_t ss, const int64_t* __restrict__ tokens,
                                 const AT* __restrict__ emb, int64_t es, int col0, AT* __restrict__ out, int64_t T,
                                 int dim) {
  const int64_t n = T * dim;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / dim;
    const int j = (int)(i - t * dim);
    stf(out + i, gelu_tanh(ldf(sg + t * ss + j)) * ldf(emb + tokens[t] * es + col0 + j));
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void side_dwa_kernel(float* __restrict__ x, const AT* __restrict__ y, int64_t ys,
                                                      const AT* __restrict__ sw, float eps, float* __restrict__ stack,
                                                      int layer, const float* __restrict__ dwa, int64_t T, int d) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  float* xr = x + t * d;
  float r = 0.f;
  if (y != nullptr) {
    float s = 0.f;
    for (int i = threadIdx.x; i < d; i += NT) {
      const float v = ldf(y + t * ys + i);
      s += v * v;
    }
    r = inv_sqrt(block_sum<NT>(s, red) / (float)d + eps);
  }
  const int64_t plane = T * d;
  for (int i = threadIdx.x; i < d; i += NT) {
    float v = xr[i];
    if (y != nullptr) v += ldf(y + t * ys + i) * r * ldf(sw + i);
    if (stack != nullptr) {
      stack[(int64_t)(layer + 1) * plane + t * d + i] = v;
      if (dwa != nullptr) {
        float a = 0.f;
        for (int j = 0; j <= layer; ++j) a += dwa[j] * stack[(int64_t)j * plane + t * d + i];
        v = a + dwa[layer + 1] * v;
      }
    }
    xr[i] = v;
  }
}

// rotate-half rotary of one element j of a `rd`-long vector v (first `dims` entries rotate, the rest pass)
template <typename AT>
__device__ __forceinline__ float rot_elem(const AT* v, int j, int dims, const float* cs) {
  const int half = dims >> 1;
  const float a = ldf(v + j);
  if (j >= dims) return a;
  if (j < half) return a * cs[j] - ldf(v + j + half) * cs[half + j];
  return a * cs[j - half] + ldf(v + j - half) * cs[j];  // cs[half + (j - half)] = sin
}

template <typename AT>
__global__ __launch_bounds__(NT) void latent_prep_kernel(const AT* __restrict__ qgd, int64_t qs, int H, int dim, int rd,
                                                         int R, int dkv_off, const AT* __restrict__ dkv_w, float eps,
                                                         const int64_t* __restrict__ positions,
                                                         const float* __restrict__ cos_sin, int dims,
                                                         AT* __restrict__ cache, AT* __restrict__ cache_t,
                                                         int page, const int64_t* __restrict__ slots,
                                                         AT* __restrict__ q_rot) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const AT* row = qgd + t * qs;
  const float* cs = cos_sin + positions[t] * dims;
  for (int i = threadIdx.x; i < H * rd; i += NT) {
    const int h = i / rd, j = i - h * rd;
    stf(q_rot + (t * H + h) * rd + j, rot_elem(row + (int64_t)h * (dim + rd) + dim, j, dims, cs));
  }
  if (dkv_off < 0) return;
  const int64_t slot = slots[t];
  const AT* lat = row + dkv_off;
  float s = 0.f;
  for (int i = threadIdx.x; i < R; i += NT) {
    const float v = ldf(lat + i);
    s += v * v;
  }
  const float r = inv_sqrt(block_sum<NT>(s, red) / (float)R + eps);
  if (slot < 0) return;
  AT* dst = cache + slot * (R + rd);
  // the latent part a second time, page-wise transposed [page][dim][token in page]: the MFMA attention kernel reads
  // its value operand (contraction over keys) from it with 16-byte loads
  AT* dst_t = cache_t != nullptr ? cache_t + (slot / page) * (int64_t)R * page + (slot % page) : nullptr;
  for (int i = threadIdx.x; i < R; i += NT) {
    const float v = ldf(lat + i) * r * ldf(dkv_w + i);
    stf(dst + i, v);
    if (dst_t != nullptr) stf(dst_t + (int64_t)i * page, v);
  }
  for (int j = threadIdx.x; j < rd; j += NT) stf(dst + R + j, rot_elem(lat + R, j, dims, cs));
}

template <typename AT>
__global__ void sigmoid_mul_kernel(const AT* __restrict__ a, int64_t a_h, int64_t a_t, const AT* __restrict__ g,
                                   int64_t gs, AT* __restrict__ out, int64_t T, int H, int vd) {
  const int64_t n = T * H * vd;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / (H * vd);
    const int c = (int)(i - t * H * vd);
    const int h = c / vd, j = c - h * vd;
    stf(out + i, ldf(a + h * a_h + t * a_t + j) * sigmoidf(ldf(g + t * gs + c)));
  }
}

// ---- latent attention ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_allsum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// One wave per (row t, group of RPW heads). Lane l holds dimensions l, l + 64, ... of the query rows, of the key row
// being visited and of the output accumulators; a key row is loaded once for the wave's heads, and its latent part
// is also the value row. Keys are visited in order first visible .. position, KB at a time, whatever the step's batch:
// a row's result does not depend on what else runs. window > 0: the row sees the last `window` keys up to its own
// position only. sink != nullptr: head h's softmax denominator also holds e^(sink[h]) (the running maximum and sum
// start from that term instead of from nothing).
template <typename AT, int MAXC, int RPW, int KB>
__global__ __launch_bounds__(256) void latent_attn_kernel(const AT* __restrict__ q_lat, int64_t ql_h, int64_t ql_t,
                                                          const AT* __restrict__ q_rot, int64_t qr_t, int64_t qr_h,
                                                          const AT* __restrict__ cache, int page, int R, int rd,
                                                          const int* __restrict__ bt, int bt_stride,
                                                          const int* __restrict__ tok_seg,
                                                          const int64_t* __restrict__ positions, float scale_log2e,
                                                          AT* __restrict__ out, int64_t o_h, int64_t o_t, int T, int H,
                                                          int n_hg, int window, const float* __restrict__ sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t task = (int64_t)blockIdx.x * 4 + wave;
  if (task >= (int64_t)T * n_hg) return;
  const int t = (int)(task / n_hg), hg = (int)(task - (int64_t)t * n_hg);
  const int h0 = hg * RPW;
  const int nh = min(RPW, H - h0);
  const int Dk = R + rd;
  float q[RPW][MAXC], acc[RPW][MAXC], m[RPW], l[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
    if (sink != nullptr && r < nh) {
      m[r] = sink[h0 + r] * 1.4426950408889634f;
      l[r] = 1.f;
    }
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int dim = lane + 64 * c;
      float v = 0.f;
      if (r < nh && dim < Dk)
        v = dim < R ? ldf(q_lat + (int64_t)(h0 + r) * ql_h + (int64_t)t * ql_t + dim)
                    : ldf(q_rot + (int64_t)t * qr_t + (int64_t)(h0 + r) * qr_h + (dim - R));
      q[r][c] = v * scale_log2e;
      acc[r][c] = 0.f;
    }
  }
  const int nkeys = (int)positions[t] + 1;
  const int* btr = bt + (int64_t)tok_seg[t] * bt_stride;
  const int jlo = window > 0 ? max(0, nkeys - window) : 0;
  for (int j0 = jlo; j0 < nkeys; j0 += KB) {
    float k[KB][MAXC];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int j = min(j0 + kb, nkeys - 1);
      const int64_t slot = (int64_t)btr[j / page] * page + (j % page);
      const AT* kr = cache + slot * Dk;
#pragma unroll
      for (int c = 0; c < MAXC; ++c) {
        const int dim = lane + 64 * c;
        k[kb][c] = dim < Dk ? ldf(kr + dim) : 0.f;
      }
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      if (r < nh) {
        float s[KB];
        float mn = m[r];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          float part = 0.f;
#pragma unroll
          for (int c = 0; c < MAXC; ++c) part += q[r][c] * k[kb][c];
          s[kb] = wave_allsum(part);
          if (j0 + kb >= nkeys) s[kb] = -INFINITY;
          mn = fmaxf(mn, s[kb]);
        }
        const float corr = fast_exp2(m[r] - mn);  // 0 on the first block (m = -inf, mn finite)
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          s[kb] = fast_exp2(s[kb] - mn);
          psum += s[kb];
        }
        l[r] = l[r] * corr + psum;
        m[r] = mn;
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
          float a = acc[r][c] * corr;
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) a += s[kb] * k[kb][c];
          acc[r][c] = a;
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    if (r < nh) {
      const float inv = 1.0f / l[r];
#pragma unroll
      for (int c = 0; c < MAXC; ++c) {
        const int dim = lane + 64 * c;
        if (dim < R) stf(out + (int64_t)(h0 + r) * o_h + (int64_t)t * o_t + dim, acc[r][c] * inv);
      }
    }
  }
}


// ---- latent attention on the matrix cores (bf16) -------------------------------------------------------------------
// One workgroup (4 waves) per tile of 32 query rows = (token, head) pairs that read the same sequence: all heads of
// floor(32 / H) consecutive tokens of a segment, or 32 heads of one token. Keys go by in blocks of 128:
//   scores   wave w takes keys 32 w .. 32 w + 31 of the block: S = Q K^T as Dk / 16 MFMA steps (32x32x16), the Q tile
//            read from LDS, the key rows straight from the paged cache (lane = key, 16 bytes per step);
//   softmax  row maxima within the wave by lane exchange and across the four waves through LDS; P = 2^(S - m) goes to
//            LDS as bf16; the row sums stay per lane and are combined once at the end;
//   values   wave w owns output columns [32 TW w, 32 TW (w + 1)) of the latent: O += P V with V read from the
//            page-transposed latent copy (lane = column, 8 consecutive keys = 16 bytes), one page per MFMA step.
// Scores, maxima, sums and the accumulators are fp32. Needs 16-token pages, kv_rank % 32 == 0, rot_dim % 16 == 0.
constexpr int MFMA_PG = 2048;  // pages of a tile's sequence staged in LDS (32k tokens; later pages read the table)

template <int TW, int NKSC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void latent_attn_mfma_kernel(
    const bf16* __restrict__ q_lat, int64_t ql_h, int64_t ql_t, const bf16* __restrict__ q_rot, int64_t qr_t,
    int64_t qr_h, const bf16* __restrict__ cache, const bf16* __restrict__ cache_t, int R, int rd,
    const int* __restrict__ bt, int bt_stride, const int* __restrict__ items, const int64_t* __restrict__ positions,
    float scale_log2e, bf16* __restrict__ out, int64_t o_h, int64_t o_t, int H, float* __restrict__ po,
    float* __restrict__ pml, int T, int window, const float* __restrict__ sink) {
  // window > 0: a row at position p sees the keys p - window < j <= p; the tile starts at the key block that holds
  // the first key its first row sees. sink != nullptr: head h's denominator also holds e^(sink[h]) (added once, at
  // the end here or in latent_merge).
  // gridDim.z > 1: the tile's key blocks are dealt to gridDim.z workgroups in contiguous ranges; each leaves its
  // unnormalised accumulators in po [z][H][T][R] and (row maximum, row sum) in pml [z][H][T][2] for latent_merge
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int Dk = R + rd, nks = Dk >> 4, qstride = Dk + 8;
  bf16* Qs = reinterpret_cast<bf16*>(smem);                 // [32][Dk + 8]
  bf16* Ps = Qs + 32 * qstride;                             // [32][128 + 8]
  float* mloc = reinterpret_cast<float*>(Ps + 32 * 136);    // [4][32]
  int* prow_s = reinterpret_cast<int*>(mloc + 128);         // [32]
  int* pg_s = prow_s + 32;                                  // [MFMA_PG]: the tile's first pages (no dependent
                                                            // global load of the block table in front of a key load)
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, lr = lane & 31, lh = lane >> 5;
  const int t0 = items[4 * blockIdx.x], ntok = items[4 * blockIdx.x + 1], sg = items[4 * blockIdx.x + 2];
  const int h0 = blockIdx.y * 32;
  const int hpr = min(H - h0, 32);
  const int nrows = ntok * hpr;
  // stage Q (zeros for rows beyond the tile) and the rows' positions
  for (int i = threadIdx.x; i < 32 * (Dk >> 3); i += 256) {
    const int r = i / (Dk >> 3), d0 = (i - r * (Dk >> 3)) << 3;
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (r < nrows) {
      const int64_t t = t0 + r / hpr, h = h0 + r % hpr;
      v = d0 < R ? load_bf16x8(q_lat + h * ql_h + t * ql_t + d0) : load_bf16x8(q_rot + t * qr_t + h * qr_h + (d0 - R));
    }
    store_bf16x8(Qs + r * qstride + d0, v);
  }
  if (threadIdx.x < 32) prow_s[threadIdx.x] = threadIdx.x < nrows ? (int)positions[t0 + threadIdx.x / hpr] : 0;
  const int maxpos = (int)positions[t0 + ntok - 1];
  {
    const int* btg = bt + (int64_t)sg * bt_stride;
    const int np = min((maxpos >> 4) + 1, MFMA_PG);
    for (int i = threadIdx.x; i < np; i += 256) pg_s[i] = btg[i];
  }
  lds_barrier();
  int prow[16];
  float m[16], lsum[16];
  f32x16 O[TW];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    prow[i] = prow_s[(i & 3) + 8 * (i >> 2) + 4 * lh];
    m[i] = -INFINITY;
    lsum[i] = 0.f;
  }
#pragma unroll
  for (int tw = 0; tw < TW; ++tw)
#pragma unroll
    for (int i = 0; i < 16; ++i) O[tw][i] = 0.f;
  const int* btr = bt + (int64_t)sg * bt_stride;
  const int nblocks = (maxpos >> 7) + 1;
  const int kbmin = window > 0 ? max(0, (int)positions[t0] - window + 1) >> 7 : 0;
  const bf16* qrow = Qs + lr * qstride + 8 * lh;
  // this wave's key row of a block, all its 16-dim steps in flight at once (one memory round trip per block); the
  // next block's row is requested right after this block's score MFMAs, so it arrives under the softmax and the
  // value pass
  bf16x8 kf[NKSC];
  auto fetch_keys = [&](int kb) {
    const int kc = min(kb * 128 + 32 * w + lr, maxpos);  // past the tile's last position: a valid row, masked below
    const int pi = kc >> 4;
    const bf16* krow = cache + ((int64_t)(pi < MFMA_PG ? pg_s[pi] : btr[pi]) * 16 + (kc & 15)) * Dk + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < NKSC; ++ks)
      if (ks < nks) kf[ks] = load_bf16x8(krow + 16 * ks);
  };
  const int nsplit = gridDim.z;
  const int bps = (nblocks - kbmin + nsplit - 1) / nsplit;
  const int kb0 = kbmin + blockIdx.z * bps, kb1 = min(nblocks, kb0 + bps);
  if (kb0 < kb1 && kb0 * 128 + 32 * w <= maxpos) fetch_keys(kb0);
  for (int kb = kb0; kb < kb1; ++kb) {
    // ---- scores of this wave's 32 keys
    const int key = kb * 128 + 32 * w + lr;
    f32x16 S;
#pragma unroll
    for (int i = 0; i < 16; ++i) S[i] = 0.f;
    const bool any = kb * 128 + 32 * w <= maxpos;  // (uniform per wave)
    if (any) {
#pragma unroll
      for (int ks = 0; ks < NKSC; ++ks)
        if (ks < nks) S = mfma32(load_bf16x8(qrow + 16 * ks), kf[ks], S);
    }
    if (kb + 1 < kb1 && (kb + 1) * 128 + 32 * w <= maxpos) fetch_keys(kb + 1);
    float s[16], mx[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = (any && key <= prow[i] && (window == 0 || key > prow[i] - window)) ? S[i] * scale_log2e : -INFINITY;
      float v = s[i];
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
      mx[i] = v;
    }
    if (lr == 0) {
#pragma unroll
      for (int i = 0; i < 16; ++i) mloc[w * 32 + (i & 3) + 8 * (i >> 2) + 4 * lh] = mx[i];
    }
    lds_barrier();
    float corr[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = (i & 3) + 8 * (i >> 2) + 4 * lh;
      const float mn = fmaxf(fmaxf(m[i], fmaxf(mloc[r], mloc[32 + r])), fmaxf(mloc[64 + r], mloc[96 + r]));
      // first block: m = -inf -> corr 0. A later split's range may start past a row's position: then mn is still
      // -inf and the row stays empty (the guards keep inf - inf out)
      corr[i] = mn == -INFINITY ? 0.f : fast_exp2(m[i] - mn);
      const float p = mn == -INFINITY ? 0.f : fast_exp2(s[i] - mn);
      lsum[i] = lsum[i] * corr[i] + p;
      m[i] = mn;
      Ps[r * 136 + 32 * w + lr] = (bf16)p;
    }
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int i = 0; i < 16; ++i) O[tw][i] *= corr[i];
    lds_barrier();
    // ---- values: one page (16 keys) per step
#pragma unroll
    for (int k0 = 0; k0 < 8; k0 += 4) {
      bf16x8 vf[4][TW];  // four pages' value operands in flight together
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        if ((kb * 8 + k0 + kk) * 16 > maxpos) break;  // (uniform) pages past the last position
        const int pi = kb * 8 + k0 + kk;
        const bf16* vp = cache_t + (int64_t)(pi < MFMA_PG ? pg_s[pi] : btr[pi]) * R * 16 + 8 * lh;
#pragma unroll
        for (int tw = 0; tw < TW; ++tw) {
          const int ct = w * TW + tw;
          if (ct * 32 < R) vf[kk][tw] = load_bf16x8(vp + (int64_t)(ct * 32 + lr) * 16);
        }
      }
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        if ((kb * 8 + k0 + kk) * 16 > maxpos) break;
        const bf16x8 a = load_bf16x8(Ps + lr * 136 + 16 * (k0 + kk) + 8 * lh);
#pragma unroll
        for (int tw = 0; tw < TW; ++tw)
          if ((w * TW + tw) * 32 < R) O[tw] = mfma32(a, vf[kk][tw], O[tw]);
      }
    }
    lds_barrier();
  }
  // ---- row sums: across the lanes of a half, then across the waves
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    float v = lsum[i];
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    lsum[i] = v;
  }
  if (lr == 0) {
#pragma unroll
    for (int i = 0; i < 16; ++i) mloc[w * 32 + (i & 3) + 8 * (i >> 2) + 4 * lh] = lsum[i];
  }
  lds_barrier();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = (i & 3) + 8 * (i >> 2) + 4 * lh;
    if (r >= nrows) continue;
    float l = mloc[r] + mloc[32 + r] + mloc[64 + r] + mloc[96 + r];
    const int64_t t = t0 + r / hpr, h = h0 + r % hpr;
    if (nsplit == 1) {
      if (sink != nullptr) l += fast_exp2(sink[h] * 1.4426950408889634f - m[i]);
      const float inv = 1.0f / l;
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) {
        const int ct = w * TW + tw;
        if (ct * 32 < R) out[h * o_h + t * o_t + ct * 32 + lr] = (bf16)(O[tw][i] * inv);
      }
    } else {
      const int64_t row = ((int64_t)blockIdx.z * H + h) * T + t;
      if (w == 0 && lr == 0) {
        pml[2 * row] = m[i];
        pml[2 * row + 1] = l;
      }
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) {
        const int ct = w * TW + tw;
        if (ct * 32 < R) po[row * R + ct * 32 + lr] = O[tw][i];
      }
    }
  }
}

// out[h][t] = sum_z 2^(m_z - m) O_z / sum_z 2^(m_z - m) l_z over the key-range splits of latent_attn_mfma_kernel
__global__ void latent_merge_kernel(const float* __restrict__ po, const float* __restrict__ pml, int nsplit, int H,
                                    int T, int R, bf16* __restrict__ out, int64_t o_h, int64_t o_t,
                                    const float* __restrict__ sink) {
  const int64_t ht = blockIdx.x;  // h * T + t
  const int h = (int)(ht / T), t = (int)(ht - (int64_t)h * T);
  float mx = -INFINITY;
  for (int z = 0; z < nsplit; ++z) mx = fmaxf(mx, pml[2 * ((int64_t)z * H * T + ht)]);
  float den = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float mz = pml[2 * ((int64_t)z * H * T + ht)];
    if (mz != -INFINITY) den += fast_exp2(mz - mx) * pml[2 * ((int64_t)z * H * T + ht) + 1];
  }
  if (sink != nullptr) den += fast_exp2(sink[h] * 1.4426950408889634f - mx);
  const float inv = 1.0f / den;
  for (int d = threadIdx.x; d < R; d += blockDim.x) {
    float a = 0.f;
    for (int z = 0; z < nsplit; ++z) {
      const float mz = pml[2 * ((int64_t)z * H * T + ht)];
      if (mz != -INFINITY) a += fast_exp2(mz - mx) * po[((int64_t)z * H * T + ht) * R + d];
    }
    out[(int64_t)h * o_h + (int64_t)t * o_t + d] = (bf16)(a * inv);
  }
}

// ---- Mamba-2 ---------------------------------------------------------------------------------------------------------
// out = act(b + sum_k w[:, k] u_(t - taps + 1 + k)) (+ u_t): b may be null, act = silu or none
template <typename AT>
__global__ void short_conv_kernel(const AT* __restrict__ proj, int64_t ps, int c0, const AT* __restrict__ w,
                                  const AT* __restrict__ b, int C, int taps, const int* __restrict__ tok_seg,
                                  const int* __restrict__ seg, const AT* __restrict__ state, AT* __restrict__ out,
                                  int64_t T, int silu, int residual) {
  const int64_t n = T * C;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / C;
    const int c = (int)(i - t * C);
    const int sg = tok_seg[t];
    const int q0 = seg[4 * sg], p0 = seg[4 * sg + 2], slot = seg[4 * sg + 3];
    float a = b ? ldf(b + c) : 0.f;
    float own = 0.f;
    for (int k = 0; k < taps; ++k) {
      const int64_t src = t - (taps - 1 - k);
      float u = 0.f;
      if (src >= q0) {
        u = ldf(proj + src * ps + c0 + c);
      } else if (p0 > 0) {
        const int si = taps - 1 + (int)(src - q0);  // the slot's tail holds the inputs before the segment
        if (si >= 0) u = ldf(state + ((int64_t)slot * (taps - 1) + si) * C + c);
      }
      a += u * ldf(w + (int64_t)c * taps + k);
      own = u;
    }
    if (silu) a = a / (1.0f + expf(-a));
    if (residual) a += own;
    stf(out + i, a);
  }
}

// the slot's tail <- the last taps - 1 entries of (old tail ++ the segment's raw inputs); one thread per (segment,
// channel) reads all it needs before it writes
template <typename AT>
__global__ void conv_state_kernel(const AT* __restrict__ proj, int64_t ps, int c0, int C, int taps,
                                  const int* __restrict__ seg, AT* __restrict__ state, int R) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)R * C) return;
  const int r = (int)(i / C), c = (int)(i - (int64_t)r * C);
  const int q0 = seg[4 * r], n = seg[4 * r + 1], p0 = seg[4 * r + 2], slot = seg[4 * r + 3];
  AT* st = state + (int64_t)slot * (taps - 1) * C + c;
  AT v[16];
  for (int k = 0; k < taps - 1; ++k) {
    const int at = n + k;  // index in (old tail ++ inputs)
    if (at < taps - 1)
      v[k] = p0 > 0 ? st[(int64_t)at * C] : (AT)0.f;
    else
      v[k] = proj[(int64_t)(q0 + at - (taps - 1)) * ps + c0 + c];
  }
  for (int k = 0; k < taps - 1; ++k) st[(int64_t)k * C] = v[k];
}

// The recurrence S_t = dA_t S_{t-1} + B_t (dt_t x_t)^T, y_t = S_t^T C_t + D x_t of one (segment, head, slice of the
// head's columns). Thread (tn, tp) keeps an RN x RP block of the state in registers (rows n = tn RN + i, columns
// p = tp RP + j), so a token costs RN + RN + RP LDS reads for 2 RN RP multiply-adds. The inputs of TB tokens (B, C, x,
// dt, dA = exp(-exp(A_log) dt)) are staged in LDS, double buffered: the next block's global loads are in flight while
// this block's tokens are scanned. Each thread's partial y (over its RN rows) goes to LDS and is summed over the TN
// row groups once per block. A head's columns are independent of each other, so a head may be cut into slices that
// run as separate workgroups (more workgroups when a step has few sequences).
constexpr int SCAN_MAXL = 24;  // staged elements a thread fetches per block, at most

template <typename AT, int RN, int RP, int TB>
__global__ __launch_bounds__(256) void ssm_scan_kernel(const AT* __restrict__ xbc, int64_t xs, const AT* __restrict__ proj, int64_t ps,
                                int dt_off, const float* __restrict__ dt_bias, const float* __restrict__ A_log,
                                const float* __restrict__ Dp, int heads, int P, int N, int G, int TN, int TP, int NPS,
                                const int* __restrict__ seg, float* __restrict__ state,
                                float* __restrict__ y, int64_t ys) {
  extern __shared__ float sm[];
  const int nthr = blockDim.x, tid = threadIdx.x;
  const int W = TP * RP;
  int b = blockIdx.x;
  const int psl = b % NPS;
  b /= NPS;
  const int h = b % heads, sgi = b / heads;
  const int q0 = seg[4 * sgi], n = seg[4 * sgi + 1], p0s = seg[4 * sgi + 2], slot = seg[4 * sgi + 3];
  const int tp = tid % TP, tn = tid / TP;
  const bool active = tn < TN;
  const int pbase = psl * W, pw = min(W, P - pbase);
  const int grp = h / (heads / G), inner = heads * P;
  float S[RN][RP];
  float* st = state + ((int64_t)slot * heads + h) * N * P;
#pragma unroll
  for (int i = 0; i < RN; ++i)
#pragma unroll
    for (int j = 0; j < RP; ++j) {
      const int nn = tn * RN + i, pp = tp * RP + j;
      S[i][j] = (active && p0s > 0 && nn < N && pp < pw) ? st[(int64_t)nn * P + pbase + pp] : 0.f;
    }
  const float A = -expf(A_log[h]), bias = dt_bias[h], Dh = Dp[h];
  const int NP = TN * RN;               // state rows padded to whole thread blocks: the pad's B and C stay zero in LDS,
                                        // so the token loop has no bounds tests
  const int stride = 2 * NP + W + 2;    // per token: B[NP] | C[NP] | x[W] | dt | dA
  const int per_tok = 2 * N + W + 1;    // fetched per token (dA is derived)
  const int bufsz = TB * stride;        // two staging buffers at sm[0], sm[bufsz] (plain offsets into the LDS array:
                                        // a pointer array would decay to generic pointers and flat loads)
  const int ypo = 2 * bufsz;            // yp [TB][TN][W] at sm[ypo]
  if (NP != N)
    for (int i = tid; i < 2 * TB * stride; i += nthr) sm[i] = 0.f;
  // what this thread fetches of every block, fixed for the whole scan: per slot the source address at block 0, its
  // step per token (a row of xbc or of proj), the LDS offset it lands at, and the token it belongs to - so a fetch is
  // one multiply-add and a load, a stash one store (the step-size slot also derives dA)
  const AT* fsrc[SCAN_MAXL];
  int fdst[SCAN_MAXL], ftok[SCAN_MAXL];  // ftok: token in block | 1 << 28 zero column | 1 << 29 step-size slot
#pragma unroll
  for (int l = 0; l < SCAN_MAXL; ++l) {
    const int e = tid + l * nthr;
    const int tt = e / per_tok, idx = e - tt * per_tok;
    const int64_t row = q0 + tt;
    const AT* xr = xbc + row * xs;
    int flags = 0;
    if (idx < N) {
      fsrc[l] = xr + inner + grp * N + idx;
      fdst[l] = idx;
    } else if (idx < 2 * N) {
      fsrc[l] = xr + inner + (G + grp) * N + (idx - N);
      fdst[l] = NP + (idx - N);
    } else if (idx < 2 * N + W) {
      const int pp = idx - 2 * N;
      fsrc[l] = xr + h * P + pbase + min(pp, pw - 1);
      fdst[l] = 2 * NP + pp;
      if (pp >= pw) flags = 1 << 28;
    } else {
      fsrc[l] = proj + row * ps + dt_off + h;
      fdst[l] = 2 * NP + W;
      flags = 1 << 29;
    }
    fdst[l] += tt * stride;
    ftok[l] = tt >= TB ? (1 << 27) : (tt | flags);  // beyond the block: never fetched
  }
  float pre[SCAN_MAXL];
  auto fetch = [&](int t0) {
    const int nt = min(TB, n - t0);
#pragma unroll
    for (int l = 0; l < SCAN_MAXL; ++l) {
      if ((ftok[l] & 0xffffff) < nt && !(ftok[l] & (1 << 27))) {
        const int64_t step = (ftok[l] & (1 << 29)) ? ps : xs;
        pre[l] = ldf(fsrc[l] + (int64_t)t0 * step);
      }
    }
  };
  auto stash = [&](int dsto, int t0) {
    const int nt = min(TB, n - t0);
#pragma unroll
    for (int l = 0; l < SCAN_MAXL; ++l) {
      if ((ftok[l] & 0xffffff) < nt && !(ftok[l] & (1 << 27))) {
        if (ftok[l] & (1 << 29)) {
          const float raw = pre[l] + bias;
          const float dt = raw > 20.f ? raw : log1pf(expf(raw));  // softplus
          sm[dsto + fdst[l]] = dt;
          sm[dsto + fdst[l] + 1] = expf(A * dt);
        } else {
          sm[dsto + fdst[l]] = (ftok[l] & (1 << 28)) ? 0.f : pre[l];
        }
      }
    }
  };
  lds_barrier();  // (the zero fill)
  fetch(0);
  stash(0, 0);
  lds_barrier();
  int it = 0;
  for (int t0 = 0; t0 < n; t0 += TB, ++it) {
    const int cur = (it & 1) * bufsz;
    const int nt = min(TB, n - t0);
    const bool more = t0 + TB < n;
    if (more) fetch(t0 + TB);  // in flight during the scan below
    if (active) {
      // the block's tokens fully unrolled, the partial outputs kept in registers until the end: no LDS store
      // sits between the tokens' LDS reads, so the reads of later tokens are issued under the arithmetic of earlier
      // ones (one wave per SIMD has nothing else to hide LDS latency with)
      float accs[TB][RP];
#pragma unroll
      for (int tt = 0; tt < TB; ++tt) {
        if (tt < nt) {
          const float* r = sm + cur + tt * stride;
          const float dt = r[2 * NP + W], dA = r[2 * NP + W + 1];
          float dx[RP], Bv[RN], Cv[RN];
#pragma unroll
          for (int j = 0; j < RP; ++j) {
            dx[j] = dt * r[2 * NP + tp * RP + j];
            accs[tt][j] = 0.f;
          }
#pragma unroll
          for (int i = 0; i < RN; ++i) {
            Bv[i] = r[tn * RN + i];
            Cv[i] = r[NP + tn * RN + i];
          }
#pragma unroll
          for (int i = 0; i < RN; ++i)
#pragma unroll
            for (int j = 0; j < RP; ++j) {
              S[i][j] = dA * S[i][j] + Bv[i] * dx[j];
              accs[tt][j] += S[i][j] * Cv[i];
            }
        }
      }
#pragma unroll
      for (int tt = 0; tt < TB; ++tt)
        if (tt < nt) {
#pragma unroll
          for (int j = 0; j < RP; ++j) sm[ypo + (tt * TN + tn) * W + tp * RP + j] = accs[tt][j];
        }
    }
    lds_barrier();
    for (int e = tid; e < nt * pw; e += nthr) {
      const int tt = e / pw, pp = e - tt * pw;
      float s = 0.f;
#pragma unroll 8
      for (int g = 0; g < TN; ++g) s += sm[ypo + (tt * TN + g) * W + pp];
      y[(int64_t)(q0 + t0 + tt) * ys + h * P + pbase + pp] = s + Dh * sm[cur + tt * stride + 2 * NP + pp];
    }
    if (more) stash(bufsz - cur, t0 + TB);
    lds_barrier();
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < RN; ++i)
#pragma unroll
      for (int j = 0; j < RP; ++j) {
        const int nn = tn * RN + i, pp = tp * RP + j;
        if (nn < N && pp < pw) st[(int64_t)nn * P + pbase + pp] = S[i][j];
      }
  }
}

// The recurrence for a step of single tokens (every segment one row: a decode step): one workgroup per (segment,
// head) streams the head's state through once - thread (g, p) owns column p and the rows n = g, g + NG, ... (the
// state's rows are read and written as consecutive columns: coalesced) - and the NG partial outputs per column are
// summed through LDS. No staging, no token loop: the state traffic is the whole cost.
template <typename AT>
__global__ __launch_bounds__(256) void ssm_step_kernel(const AT* __restrict__ xbc, int64_t xs,
                                                       const AT* __restrict__ proj, int64_t ps, int dt_off,
                                                       const float* __restrict__ dt_bias,
                                                       const float* __restrict__ A_log, const float* __restrict__ Dp,
                                                       int heads, int P, int N, int G, int NG,
                                                       const int* __restrict__ seg, float* __restrict__ state,
                                                       float* __restrict__ y, int64_t ys) {
  __shared__ float part[256];
  const int sgi = blockIdx.x / heads, h = blockIdx.x - sgi * heads;
  const int64_t row = seg[4 * sgi];
  const int p0s = seg[4 * sgi + 2], slot = seg[4 * sgi + 3];
  const int tid = threadIdx.x, p = tid % P, g = tid / P;
  const int grp = h / (heads / G), inner = heads * P;
  const float raw = ldf(proj + row * ps + dt_off + h) + dt_bias[h];
  const float dt = raw > 20.f ? raw : log1pf(expf(raw));
  const float dA = expf(-expf(A_log[h]) * dt);
  const AT* xr = xbc + row * xs;
  const float xv = ldf(xr + h * P + p), dx = dt * xv;
  const AT* Br = xr + inner + grp * N;
  const AT* Cr = Br + (int64_t)G * N;
  float* st = state + ((int64_t)slot * heads + h) * N * P + p;
  float acc = 0.f;
  if (p0s > 0) {
#pragma unroll 4
    for (int nn = g; nn < N; nn += NG) {
      const float sv = dA * st[(int64_t)nn * P] + ldf(Br + nn) * dx;
      st[(int64_t)nn * P] = sv;
      acc += sv * ldf(Cr + nn);
    }
  } else {  // first token of its sequence: the slot is written, not read
#pragma unroll 4
    for (int nn = g; nn < N; nn += NG) {
      const float sv = ldf(Br + nn) * dx;
      st[(int64_t)nn * P] = sv;
      acc += sv * ldf(Cr + nn);
    }
  }
  part[tid] = acc;
  __syncthreads();
  if (g == 0) {
    float s = 0.f;
    for (int gg = 0; gg < NG; ++gg) s += part[gg * P + p];
    y[row * ys + h * P + p] = s + Dp[h] * xv;
  }
}

// Chunk-parallel scan, middle pass. A long segment is cut into chunks that are first scanned independently from a
// zero state (ssm_scan over the chunk table `vseg`); here the chunks' entry states are rebuilt in order,
//   S_in[0] = the sequence's state (zero at position 0),  S_in[c + 1] = D_c S_in[c] + S_loc[c],
// with D_c = exp(-exp(A_log) sum of the chunk's step sizes), S_in[c] replaces S_loc[c] in the chunk's scratch slot (the
// second scan starts from it) and the value after the last chunk is the sequence's new state. One workgroup per
// (segment, head); cs[s] = (first chunk, chunks, first position, state slot).
template <typename AT>
__global__ __launch_bounds__(256) void ssm_combine_kernel(const AT* __restrict__ proj, int64_t ps, int dt_off,
                                                          const float* __restrict__ dt_bias,
                                                          const float* __restrict__ A_log, int heads, int NP_,
                                                          const int* __restrict__ vseg, const int* __restrict__ cs,
                                                          float* __restrict__ tmp, float* __restrict__ state) {
  __shared__ float red[4];
  __shared__ float D[256];
  const int sgi = blockIdx.x / heads, h = blockIdx.x - sgi * heads;
  const int c0 = cs[4 * sgi], nch = cs[4 * sgi + 1], p0 = cs[4 * sgi + 2], slot = cs[4 * sgi + 3];
  const float A = -expf(A_log[h]), bias = dt_bias[h];
  for (int c = 0; c < nch; ++c) {
    const int q0 = vseg[4 * (c0 + c)], n = vseg[4 * (c0 + c) + 1];
    float sdt = 0.f;
    for (int t = threadIdx.x; t < n; t += 256) {
      const float raw = ldf(proj + (int64_t)(q0 + t) * ps + dt_off + h) + bias;
      sdt += raw > 20.f ? raw : log1pf(expf(raw));
    }
    sdt = block_sum<256>(sdt, red);
    if (threadIdx.x == 0) D[c] = expf(A * sdt);
  }
  __syncthreads();
  float* st = state + ((int64_t)slot * heads + h) * NP_;
  for (int e = threadIdx.x; e < NP_; e += 256) {
    float sv = p0 > 0 ? st[e] : 0.f;
    for (int c = 0; c < nch; ++c) {
      float* tp = tmp + ((int64_t)vseg[4 * (c0 + c) + 3] * heads + h) * NP_ + e;
      const float loc = *tp;
      *tp = sv;
      sv = D[c] * sv + loc;
    }
    st[e] = sv;
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void gated_norm_kernel(const float* __restrict__ y, int64_t ys, const AT* __restrict__ z,
                                                        int64_t zs, const AT* __restrict__ w, int gs, float eps,
                                                        AT* __restrict__ out, int64_t os) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int c0 = blockIdx.y * gs;
  float s = 0.f;
  for (int i = threadIdx.x; i < gs; i += NT) {
    const float zv = ldf(z + t * zs + c0 + i);
    const float v = y[t * ys + c0 + i] * (zv / (1.0f + expf(-zv)));
    s += v * v;
  }
  const float r = inv_sqrt(block_sum<NT>(s, red) / (float)gs + eps);
  for (int i = threadIdx.x; i < gs; i += NT) {
    const float zv = ldf(z + t * zs + c0 + i);
    const float v = y[t * ys + c0 + i] * (zv / (1.0f + expf(-zv)));
    stf(out + t * os + c0 + i, v * r * ldf(w + c0 + i));
  }
}

static inline int ew_grid(int64_t n) { return (int)std::min<int64_t>((n + 255) / 256, 65535 * 4); }

}  // namespace hy
}  // namespace kafka

using namespace kafka::hy;

#define DISPATCH_AT(f32, ...)             \
  if (f32) {                              \
    using AT = float;                     \
    __VA_ARGS__;                          \
  } else {                                \
    using AT = bf16;                      \
    __VA_ARGS__;                          \
  }

extern "C" {

hipError_t kafka_hy_ln_shift(int f32, const float* x, int64_t xs, const void* w, const void* b, float eps, void* out,
                             int64_t os, int T, int d, const void* mu, const int* tok_seg, const int* seg,
                             const float* state, float* last, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  DISPATCH_AT(f32, {
    auto a = [&](auto k) {
      k<<<T, NT, 0, st>>>(x, xs, (const AT*)w, (const AT*)b, eps, (AT*)out, os, d, (const AT*)mu, tok_seg, seg, state,
                          last);
    };
    if (d <= 4 * NT) a(ln_shift_reg_kernel<AT, 4>);
    else if (d <= 16 * NT) a(ln_shift_reg_kernel<AT, 16>);
    else a(ln_shift_kernel<AT>);
  });
  return hipGetLastError();
}

hipError_t kafka_hy_scatter_rows(float* dst, const int* seg, const float* src, int R, int d, hipStream_t st) {
  if (R <= 0) return hipSuccess;
  scatter_rows_kernel<<<R, 256, 0, st>>>(dst, seg, src, d);
  return hipGetLastError();
}

hipError_t kafka_hy_add_ln(int f32, float* x, int64_t xs, const void* y, int64_t ys, const void* w, const void* b,
                           float eps, int T, int d, void* out2, int64_t os, const void* w2, const void* b2,
                           hipStream_t st) {
  if (T <= 0) return hipSuccess;
  const int mode = out2 == nullptr ? 0 : (w2 != nullptr ? 1 : 2);
  DISPATCH_AT(f32, {
    auto a = [&](auto k) {
      k<<<T, NT, 0, st>>>(x, xs, (const AT*)y, ys, (const AT*)w, (const AT*)b, eps, d, (AT*)out2, os, (const AT*)w2,
                          (const AT*)b2);
    };
    if (d <= 4 * NT) {
      if (mode == 0) a(add_ln_reg_kernel<AT, 4, 0>);
      else if (mode == 1) a(add_ln_reg_kernel<AT, 4, 1>);
      else a(add_ln_reg_kernel<AT, 4, 2>);
    } else if (d <= 16 * NT) {
      if (mode == 0) a(add_ln_reg_kernel<AT, 16, 0>);
      else if (mode == 1) a(add_ln_reg_kernel<AT, 16, 1>);
      else a(add_ln_reg_kernel<AT, 16, 2>);
    } else if (mode == 0) a(add_ln_kernel<AT, 0>);
    else if (mode == 1) a(add_ln_kernel<AT, 1>);
    else a(add_ln_kernel<AT, 2>);
  });
  return hipGetLastError();
}

hipError_t kafka_hy_gelu_mul(int f32, const void* gu, int64_t gs, void* out, int64_t T, int F, hipStream_t st) {
  if (T * F <= 0) return hipSuccess;
  DISPATCH_AT(f32, gelu_mul_kernel<AT><<<ew_grid(T * F), 256, 0, st>>>((const AT*)gu, gs, (AT*)out, T, F));
  return hipGetLastError();
}

hipError_t kafka_hy_side_gate(int f32, const void* sg, int64_t ss, const int64_t* tokens, const void* emb, int64_t es,
                              int col0, void* out, int64_t T, int dim, hipStream_t st) {
  if (T * dim <= 0) return hipSuccess;
  DISPATCH_AT(f32, side_gate_kernel<AT><<<ew_grid(T * dim), 256, 0, st>>>((const AT*)sg, ss, tokens, (const AT*)emb,
                                                                          es, col0, (AT*)out, T, dim));
  return hipGetLastError();
}

hipError_t kafka_hy_side_dwa(int f32, float* x, const void* y, int64_t ys, const void* sw, float eps, float* stack,
                             int layer, const float* dwa, int64_t T, int d, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  DISPATCH_AT(f32, {
    auto a = [&](auto k) { k<<<(int)T, NT, 0, st>>>(x, (const AT*)y, ys, (const AT*)sw, eps, stack, layer, dwa, T, d); };
    if (d <= 4 * NT) a(side_dwa_reg_kernel<AT, 4>);
    else if (d <= 16 * NT) a(side_dwa_reg_kernel<AT, 16>);
    else a(side_dwa_kernel<AT>);
  });
  return hipGetLastError();
}

hipError_t kafka_hy_latent_prep(int f32, const void* qgd, int64_t qs, int T, int H, int dim, int rd, int R, int dkv_off,
                                const void* dkv_w, float eps, const int64_t* positions, const float* cos_sin, int dims,
                                void* cache, void* cache_t, int page, const int64_t* slots, void* q_rot,
                                hipStream_t st) {
  if (T <= 0) return hipSuccess;
  DISPATCH_AT(f32, latent_prep_kernel<AT><<<T, NT, 0, st>>>((const AT*)qgd, qs, H, dim, rd, R, dkv_off,
                                                           (const AT*)dkv_w, eps, positions, cos_sin, dims, (AT*)cache,
                                                           (AT*)cache_t, page, slots, (AT*)q_rot));
  return hipGetLastError();
}

hipError_t kafka_hy_sigmoid_mul(int f32, const void* a, int64_t a_h, int64_t a_t, const void* g, int64_t gs, void* out,
                                int64_t T, int H, int vd, hipStream_t st) {
  if (T * H * vd <= 0) return hipSuccess;
  DISPATCH_AT(f32, sigmoid_mul_kernel<AT><<<ew_grid(T * H * vd), 256, 0, st>>>((const AT*)a, a_h, a_t, (const AT*)g,
                                                                                gs, (AT*)out, T, H, vd));
  return hipGetLastError();
}

// largest key-row length (latent + rotary part) the attention kernel holds in registers
int kafka_hy_latent_attn_max_dk() { return 640; }

hipError_t kafka_hy_latent_attn(int f32, const void* q_lat, int64_t ql_h, int64_t ql_t, const void* q_rot, int64_t qr_t,
                                int64_t qr_h, const void* cache, int page, int R, int rd, const int* bt, int bt_stride,
                                const int* tok_seg, const int64_t* positions, float scale, void* out, int64_t o_h,
                                int64_t o_t, int T, int H, int window, const float* sink, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (window < 0) return hipErrorInvalidValue;
  constexpr int RPW = 4;
  const int n_hg = (H + RPW - 1) / RPW;
  const int64_t tasks = (int64_t)T * n_hg;
  const int grid = (int)((tasks + 3) / 4);
  const float sl = scale * 1.4426950408889634f;
  const int Dk = R + rd;
  DISPATCH_AT(f32, {
    auto a = [&](auto k) {
      k<<<grid, 256, 0, st>>>((const AT*)q_lat, ql_h, ql_t, (const AT*)q_rot, qr_t, qr_h, (const AT*)cache, page, R, rd,
                              bt, bt_stride, tok_seg, positions, sl, (AT*)out, o_h, o_t, T, H, n_hg, window, sink);
    };
    if (Dk <= 192) a(latent_attn_kernel<AT, 3, RPW, 4>);
    else if (Dk <= 384) a(latent_attn_kernel<AT, 6, RPW, 4>);
    else if (Dk <= 640) a(latent_attn_kernel<AT, 10, RPW, 2>);
    else return hipErrorInvalidValue;
  });
  return hipGetLastError();
}

// bf16 shapes the matrix-core kernel takes (else the per-wave kernel above runs)
int kafka_hy_latent_mfma_ok(int page, int R, int rd) {
  return page == 16 && R % 32 == 0 && rd % 16 == 0 && R >= 32 && R <= 512 && R + rd <= 640;
}

hipError_t kafka_hy_latent_attn_mfma(const void* q_lat, int64_t ql_h, int64_t ql_t, const void* q_rot, int64_t qr_t,
                                     int64_t qr_h, const void* cache, const void* cache_t, int R, int rd,
                                     const int* bt, int bt_stride, const int* items, int n_items,
                                     const int64_t* positions, float scale, void* out, int64_t o_h, int64_t o_t, int H,
                                     int nsplit, float* po, float* pml, int T, int window, const float* sink,
                                     hipStream_t st) {
  if (n_items <= 0) return hipSuccess;
  if (window < 0) return hipErrorInvalidValue;
  if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && (po == nullptr || pml == nullptr))) return hipErrorInvalidValue;
  if (!kafka_hy_latent_mfma_ok(16, R, rd)) return hipErrorInvalidValue;
  const int Dk = R + rd;
  const size_t lds = (size_t)32 * (Dk + 8) * 2 + 32 * 136 * 2 + 128 * 4 + 32 * 4 + MFMA_PG * 4;
  const dim3 grid((unsigned)n_items, (unsigned)((H + 31) / 32), (unsigned)nsplit);
  const float sl = scale * 1.4426950408889634f;
  const int tw = (R / 32 + 3) / 4;
  auto a = [&](auto k) {
    k<<<grid, 256, lds, st>>>((const bf16*)q_lat, ql_h, ql_t, (const bf16*)q_rot, qr_t, qr_h, (const bf16*)cache,
                              (const bf16*)cache_t, R, rd, bt, bt_stride, items, positions, sl, (bf16*)out, o_h, o_t, H,
                              po, pml, T, window, sink);
  };
  const int nks = Dk / 16;
  if (tw == 1 && nks <= 12) a(latent_attn_mfma_kernel<1, 12>);
  else if (tw == 1) a(latent_attn_mfma_kernel<1, 40>);
  else if (tw == 2 && nks <= 24) a(latent_attn_mfma_kernel<2, 24>);
  else if (tw == 2) a(latent_attn_mfma_kernel<2, 40>);
  else if (tw == 3) a(latent_attn_mfma_kernel<3, 40>);
  else if (nks <= 36) a(latent_attn_mfma_kernel<4, 36>);
  else a(latent_attn_mfma_kernel<4, 40>);
  if (nsplit > 1)
    latent_merge_kernel<<<(unsigned)((int64_t)H * T), 128, 0, st>>>(po, pml, nsplit, H, T, R, (bf16*)out, o_h, o_t,
                                                                    sink);
  return hipGetLastError();
}

hipError_t kafka_hy_short_conv(int f32, const void* proj, int64_t ps, int c0, const void* w, const void* b, int C,
                               int taps, const int* tok_seg, const int* seg, int R, void* state, void* out, int64_t T,
                               int silu, int residual, hipStream_t st) {
  if (T <= 0 || C <= 0 || taps > 16 || taps < 1) return (taps > 16 || taps < 1) ? hipErrorInvalidValue : hipSuccess;
  DISPATCH_AT(f32, {
    short_conv_kernel<AT><<<ew_grid(T * C), 256, 0, st>>>((const AT*)proj, ps, c0, (const AT*)w, (const AT*)b, C, taps,
                                                          tok_seg, seg, (const AT*)state, (AT*)out, T, silu, residual);
    if (taps > 1)
      conv_state_kernel<AT><<<(int)(((int64_t)R * C + 255) / 256), 256, 0, st>>>((const AT*)proj, ps, c0, C, taps, seg,
                                                                                (AT*)state, R);
  });
  return hipGetLastError();
}

// launch shape of the scan for a head of N x P state and `work` = segments x heads workgroups before slicing:
// returns 0 when no shape fits
struct ScanPlan { int TN, TP, NPS, TB, threads; size_t lds; };
static int scan_plan(int P, int N, int64_t work, ScanPlan* sp) {
  constexpr int RN = 8, RP = 4;
  if (P < 1 || N < 1 || N > 4096 || P > 4096) return 0;
  const int TN = (N + RN - 1) / RN;
  if (TN > 256) return 0;
  int TP = std::max(1, std::min((P + RP - 1) / RP, std::max(1, 256 / TN)));
  auto slices = [&](int tp) { return (P + tp * RP - 1) / (tp * RP); };
  while (TP >= 8 && work * slices(TP) < 256) TP /= 2;  // few sequences: narrower slices, more workgroups
  const int NPS = slices(TP), W = TP * RP;
  const int threads = std::max(64, (TN * TP + 63) / 64 * 64);
  if (threads > 256) return 0;
  for (int TB = 8; TB >= 1; TB /= 2) {
    const size_t lds = sizeof(float) * ((size_t)2 * TB * (2 * TN * RN + W + 2) + (size_t)TB * TN * W);
    const int lpt = (TB * (2 * N + W + 1) + threads - 1) / threads;
    if (lds <= 60 * 1024 && lpt <= 24) {
      *sp = {TN, TP, NPS, TB, threads, lds};
      return 1;
    }
  }
  return 0;
}

int kafka_hy_scan_groups(int P, int N) {
  ScanPlan sp;
  return scan_plan(P, N, 1 << 20, &sp) ? sp.threads : 0;
}

hipError_t kafka_hy_ssm_scan(int f32, const void* xbc, int64_t xs, const void* proj, int64_t ps, int dt_off,
                             const float* dt_bias, const float* A_log, const float* Dp, int heads, int P, int N, int G,
                             const int* seg, int R, int single, float* state, float* y, int64_t ys, hipStream_t st) {
  if (R <= 0) return hipSuccess;
  if (single && P <= 256) {  // every segment one row
    const int NG = std::max(1, std::min(256 / P, N));
    DISPATCH_AT(f32, ssm_step_kernel<AT><<<R * heads, P * NG, 0, st>>>((const AT*)xbc, xs, (const AT*)proj, ps, dt_off,
                                                                      dt_bias, A_log, Dp, heads, P, N, G, NG, seg,
                                                                      state, y, ys));
    return hipGetLastError();
  }
  ScanPlan sp;
  if (!scan_plan(P, N, (int64_t)R * heads, &sp)) return hipErrorInvalidValue;
  DISPATCH_AT(f32, {
    auto a = [&](auto k) {
      k<<<R * heads * sp.NPS, sp.threads, sp.lds, st>>>((const AT*)xbc, xs, (const AT*)proj, ps, dt_off, dt_bias, A_log,
                                                        Dp, heads, P, N, G, sp.TN, sp.TP, sp.NPS, seg, state, y, ys);
    };
    if (sp.TB == 8) a(ssm_scan_kernel<AT, 8, 4, 8>);
    else if (sp.TB == 4) a(ssm_scan_kernel<AT, 8, 4, 4>);
    else if (sp.TB == 2) a(ssm_scan_kernel<AT, 8, 4, 2>);
    else a(ssm_scan_kernel<AT, 8, 4, 1>);
  });
  return hipGetLastError();
}

hipError_t kafka_hy_ssm_combine(int f32, const void* proj, int64_t ps, int dt_off, const float* dt_bias,
                                const float* A_log, int heads, int NP_, const int* vseg, const int* cs, int S,
                                float* tmp, float* state, hipStream_t st) {
  if (S <= 0) return hipSuccess;
  DISPATCH_AT(f32, ssm_combine_kernel<AT><<<S * heads, 256, 0, st>>>((const AT*)proj, ps, dt_off, dt_bias, A_log, heads,
                                                                    NP_, vseg, cs, tmp, state));
  return hipGetLastError();
}

hipError_t kafka_hy_gated_norm(int f32, const float* y, int64_t ys, const void* z, int64_t zs, const void* w, int inner,
                               int groups, float eps, void* out, int64_t os, int64_t T, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  DISPATCH_AT(f32, gated_norm_kernel<AT><<<dim3((unsigned)T, (unsigned)groups), NT, 0, st>>>(
                       y, ys, (const AT*)z, zs, (const AT*)w, inner / groups, eps, (AT*)out, os));
  return hipGetLastError();
}

}  // extern "C"
