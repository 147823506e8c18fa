// Kernels for decoders whose mixers are gated recurrences beside (or in turn with) softmax attention, for gfx950.
//
// Every kernel is built for bf16 and for fp32 activations; norm statistics, rotation, the head mix, gates, candidates,
// decays and recurrent states are fp32 in both. Sizes are run-time values with no alignment assumptions.
//
//   act_norm        RMS norm (or layer norm without bias) over a column range of activation rows, fp32 weight
//   gate_mul        a * sigmoid(gate columns) * scale into a column slice
//   mingru_scan     S <- (1 - z) S + z c per channel with z = sigmoid(.), c = u + 1/2 (u >= 0) | sigmoid(u) (u < 0),
//                   out = S silu(gate): row by row (one thread per (segment, channel), the inputs of 8 rows loaded
//                   together), or for long segments in chunks (decays and inputs in parallel over all rows, per-chunk
//                   scans from zero, entry states carried in order, per-chunk scans from the entry states)
//   hgrn2_scan      per head S <- diag(f) S + (1 - f) v^T, out = S^T silu(q), f = l + (1 - l) sigmoid(.): a workgroup per
//                   (segment, head, 64 value columns), a thread keeps a quarter of the rows of one column in registers,
//                   8 tokens' inputs staged in LDS (double buffered, the next block's loads in flight)
//   rope_kv_store   rotation of q and k heads (halves or neighbour pairs), optional mix of the queries over the heads
//                   (so that one product with the whole key row gives the head-mixed score), paged key / transposed
//                   value store
#include "common.h"

namespace kafka {
namespace hp {

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)(*p); }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

constexpr int NT = 256;
constexpr int PAGE = 16;

__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float siluf(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- norm over a column range of activation rows ---------------------------------------------------------------------
template <typename AT>
__global__ __launch_bounds__(NT) void act_norm_kernel(const AT* __restrict__ x, int64_t xs, int c0, int n,
                                                      const float* __restrict__ w, float eps, AT* __restrict__ out,
                                                      int64_t os, bool center) {
  __shared__ float red[NT / 64];
  const AT* r = x + (int64_t)blockIdx.x * xs + c0;
  float mean = 0.f;
  if (center) {
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += NT) s += ldf(r + i);
    mean = block_sum<NT>(s, red) / (float)n;
  }
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += NT) {
    const float v = ldf(r + i) - mean;
    s += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)n + eps);
  AT* o = out + (int64_t)blockIdx.x * os;
  for (int i = threadIdx.x; i < n; i += NT) stf(o + i, (ldf(r + i) - mean) * rs * w[i]);
}

template <typename AT>
__global__ void gate_mul_kernel(const AT* __restrict__ a, int64_t as, const AT* __restrict__ g, int64_t gs, int g_off,
                                float scale, AT* __restrict__ out, int64_t os, int64_t T, int n) {
  const int64_t tot = T * n;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < tot; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / n;
    const int c = (int)(i - t * n);
    stf(out + t * os + c, ldf(a + t * as + c) * sigmoidf(ldf(g + t * gs + g_off + c)) * scale);
  }
}

// the same on bf16 rows whose sizes, offsets, strides and bases are multiples of 8 elements
__global__ void gate_mul_vec8_kernel(const bf16* __restrict__ a, int64_t as, const bf16* __restrict__ g, int64_t gs,
                                     int g_off, float scale, bf16* __restrict__ out, int64_t os, int64_t T, int n) {
  const int n8 = n >> 3;
  const int64_t tot = T * n8;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < tot; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / n8;
    const int c = (int)(i - t * n8) << 3;
    const bf16x8 av = load_bf16x8(a + t * as + c), gv = load_bf16x8(g + t * gs + g_off + c);
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (bf16)((float)av[j] * sigmoidf((float)gv[j]) * scale);
    store_bf16x8(out + t * os + c, o);
  }
}

// ---- minGRU -------------------------------------------------------------------------------------------------------------
constexpr int MG_TB = 8;    // rows whose inputs are loaded together
constexpr int MG_CH = 64;   // rows of a chunk of the chunked form

// decay a = 1 - z and input b = z c of one row and channel from the two pre-activations (biases added here, fp32)
__device__ __forceinline__ void mingru_ab(float pz, float px, float& a, float& b) {
  const float z = sigmoidf(pz);
  const float c = px >= 0.f ? px + 0.5f : sigmoidf(px);
  a = 1.0f - z;
  b = z * c;
}

template <typename AT>
__global__ void mingru_scan_kernel(const AT* __restrict__ proj, int64_t ps, const float* __restrict__ bias,
                                   const int* __restrict__ seg, float* __restrict__ state, AT* __restrict__ out,
                                   int64_t os, int W) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int r = blockIdx.y;
  const int q0 = seg[4 * r], n = seg[4 * r + 1], p0 = seg[4 * r + 2], slot = seg[4 * r + 3];
  float S = p0 > 0 ? state[(int64_t)slot * W + c] : 0.f;
  const float bz = bias[c], bx = bias[W + c];
  for (int b0 = 0; b0 < n; b0 += MG_TB) {
    const int nt = min(MG_TB, n - b0);
    float pz[MG_TB], px[MG_TB], pg[MG_TB];
#pragma unroll
    for (int j = 0; j < MG_TB; ++j) {
      const int64_t t = (int64_t)q0 + b0 + (j < nt ? j : 0);
      pz[j] = ldf(proj + t * ps + c);
      px[j] = ldf(proj + t * ps + W + c);
      pg[j] = ldf(proj + t * ps + 2 * W + c);
    }
    float a[MG_TB], b[MG_TB];
#pragma unroll
    for (int j = 0; j < MG_TB; ++j) {
      mingru_ab(pz[j] + bz, px[j] + bx, a[j], b[j]);
      pg[j] = siluf(pg[j]);
    }
#pragma unroll
    for (int j = 0; j < MG_TB; ++j) {
      if (j < nt) {
        S = a[j] * S + b[j];
        stf(out + ((int64_t)q0 + b0 + j) * os + c, S * pg[j]);
      }
    }
  }
  state[(int64_t)slot * W + c] = S;
}

// chunked form, step 1: ab[t][0 .. W) = decay, ab[t][W .. 2 W) = input, for every row and channel in parallel
template <typename AT>
__global__ void mingru_prep_kernel(const AT* __restrict__ proj, int64_t ps, const float* __restrict__ bias,
                                   float* __restrict__ ab, int64_t T, int W) {
  const int64_t n = T * W;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / W;
    const int c = (int)(i - t * W);
    float a, b;
    mingru_ab(ldf(proj + t * ps + c) + bias[c], ldf(proj + t * ps + W + c) + bias[W + c], a, b);
    ab[t * 2 * W + c] = a;
    ab[t * 2 * W + W + c] = b;
  }
}

// MODE 0: the chunk's decay product and its scan from zero -> ce[((r * nch + ch) * 2 + {0, 1}) * W + c];
// MODE 1: the scan again from the entry state in ce[...][0], out = S * silu(gate)
template <typename AT, int MODE>
__global__ void mingru_chunk_kernel(const float* __restrict__ ab, const AT* __restrict__ proj, int64_t ps,
                                    const int* __restrict__ seg, int nch, float* __restrict__ ce, AT* __restrict__ out,
                                    int64_t os, int W) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ch = blockIdx.y, r = blockIdx.z;
  const int q0 = seg[4 * r], n = seg[4 * r + 1];
  if (c >= W || ch * MG_CH >= n) return;
  const int nt = min(MG_CH, n - ch * MG_CH);
  float* slot = ce + ((int64_t)(r * nch + ch) * 2) * W + c;
  float S = MODE == 1 ? slot[0] : 0.f, A = 1.f;
  for (int b0 = 0; b0 < nt; b0 += MG_TB) {
    float a[MG_TB], b[MG_TB], y[MG_TB];
#pragma unroll
    for (int j = 0; j < MG_TB; ++j) {
      const int64_t t = (int64_t)q0 + ch * MG_CH + b0 + (b0 + j < nt ? j : 0);
      a[j] = ab[t * 2 * W + c];
      b[j] = ab[t * 2 * W + W + c];
      if (MODE == 1) y[j] = ldf(proj + t * ps + 2 * W + c);
    }
    if (MODE == 1) {
#pragma unroll
      for (int j = 0; j < MG_TB; ++j) y[j] = siluf(y[j]);
    }
#pragma unroll
    for (int j = 0; j < MG_TB; ++j) {
      if (b0 + j < nt) {
        S = a[j] * S + b[j];
        if (MODE == 0) A *= a[j];
        if (MODE == 1) stf(out + ((int64_t)q0 + ch * MG_CH + b0 + j) * os + c, S * y[j]);
      }
    }
  }
  if (MODE == 0) {
    slot[0] = A;
    slot[W] = S;
  }
}

// the chunks' entry states in order; the last state is the sequence's new state
__global__ void mingru_carry_kernel(const int* __restrict__ seg, int nch, float* __restrict__ ce,
                                    float* __restrict__ state, int W) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int r = blockIdx.y;
  const int n = seg[4 * r + 1], p0 = seg[4 * r + 2], slot = seg[4 * r + 3];
  float S = p0 > 0 ? state[(int64_t)slot * W + c] : 0.f;
  const int used = (n + MG_CH - 1) / MG_CH;
  for (int ch = 0; ch < used; ++ch) {
    float* s2 = ce + ((int64_t)(r * nch + ch) * 2) * W + c;
    const float A = s2[0], B = s2[W];
    s2[0] = S;   // the chunk's entry state
    S = A * S + B;
  }
  state[(int64_t)slot * W + c] = S;
}

// ---- HGRN2 --------------------------------------------------------------------------------------------------------------
constexpr int HG_DG = 4;   // row groups (one wave each)
constexpr int HG_TB = 8;   // tokens per staged block

// One workgroup per (segment, head, 64 value columns). Thread (dg, vv) keeps rows d = dg RD .. dg RD + RD - 1 of column
// vv of the head's matrix in registers. The inputs of HG_TB tokens are staged in LDS at a time (silu(q), the forget gate
// f, the value slice), double buffered, the next block's global loads in flight while this block is scanned: the
// threads walk the block's tokens without synchronising (the matrix is thread-private), leave HG_DG partial read-outs
// per (token, column) in LDS, and after one barrier the partials are summed. Two barriers per block. Rows past D hold
// f = 1 and q = 0: their (zero) state stays zero.
template <typename AT, int RD>
__global__ __launch_bounds__(NT) void hgrn2_scan_kernel(const AT* __restrict__ proj, int64_t ps, int q_off, int f_off,
                                                        int v_off, const float* __restrict__ f_bias,
                                                        const float* __restrict__ lower, int H, int D, int Dv,
                                                        const int* __restrict__ seg, float* __restrict__ Sst,
                                                        float* __restrict__ out, int64_t os) {
  constexpr int DMAX = HG_DG * RD;
  constexpr int NQF = (2 * DMAX * HG_TB + NT - 1) / NT;   // staged q | f elements per thread
  constexpr int NV = (64 * HG_TB + NT - 1) / NT;          // staged value elements per thread
  __shared__ __attribute__((aligned(16))) float qf[2][HG_TB][2][DMAX];
  __shared__ float vs[2][HG_TB][64];
  __shared__ float part[HG_TB][HG_DG][64];
  const int r = blockIdx.z, h = blockIdx.y, v0 = blockIdx.x * 64;
  const int q0 = seg[4 * r], n = seg[4 * r + 1], p0 = seg[4 * r + 2], slot = seg[4 * r + 3];
  const int dg = threadIdx.x >> 6, vv = threadIdx.x & 63;
  const bool vok = v0 + vv < Dv;
  float S[RD];
  float* Sp = Sst + (((int64_t)slot * H + h) * D) * Dv + v0 + vv;
#pragma unroll
  for (int i = 0; i < RD; ++i) {
    const int d = dg * RD + i;
    S[i] = (p0 > 0 && d < D && vok) ? Sp[(int64_t)d * Dv] : 0.f;
  }
  const int qo = q_off + h * D, fo = f_off + h * D, vo = v_off + h * Dv + v0;
  const int nblk = (n + HG_TB - 1) / HG_TB;
  float pqf[NQF], pv[NV];
  auto fetch = [&](int blk) {   // global loads of a block into registers
    const int64_t t0 = (int64_t)q0 + blk * HG_TB;
    const int nt = min(HG_TB, n - blk * HG_TB);
#pragma unroll
    for (int e = 0; e < NQF; ++e) {
      const int idx = threadIdx.x + NT * e;
      const int j = idx / (2 * DMAX), rr = idx - j * 2 * DMAX, which = rr / DMAX, d = rr - which * DMAX;
      pqf[e] = (j < nt && d < D) ? ldf(proj + (t0 + j) * ps + (which ? fo : qo) + d) : 0.f;
    }
#pragma unroll
    for (int e = 0; e < NV; ++e) {
      const int idx = threadIdx.x + NT * e;
      const int j = idx >> 6, c = idx & 63;
      pv[e] = (j < nt && v0 + c < Dv) ? ldf(proj + (t0 + j) * ps + vo + c) : 0.f;
    }
  };
  auto stage = [&](int buf) {   // registers -> LDS (queries through silu, forget gates through their bound)
#pragma unroll
    for (int e = 0; e < NQF; ++e) {
      const int idx = threadIdx.x + NT * e;
      const int j = idx / (2 * DMAX), rr = idx - j * 2 * DMAX, which = rr / DMAX, d = rr - which * DMAX;
      if (j < HG_TB) {
        float v;
        if (d >= D) {
          v = which ? 1.0f : 0.f;
        } else if (which) {
          const float lo = lower[h * D + d];
          v = lo + (1.0f - lo) * sigmoidf(pqf[e] + f_bias[h * D + d]);
        } else {
          v = siluf(pqf[e]);
        }
        qf[buf][j][which][d] = v;
      }
    }
#pragma unroll
    for (int e = 0; e < NV; ++e) {
      const int idx = threadIdx.x + NT * e;
      if ((idx >> 6) < HG_TB) vs[buf][idx >> 6][idx & 63] = pv[e];
    }
  };
  fetch(0);
  stage(0);
  for (int blk = 0; blk < nblk; ++blk) {
    const int buf = blk & 1;
    const int nt = min(HG_TB, n - blk * HG_TB);
    if (blk + 1 < nblk) fetch(blk + 1);
    lds_barrier();     // this block's staged inputs are visible; the other buffer and `part` are free
#pragma unroll 1
    for (int j = 0; j < nt; ++j) {
      const float v = vs[buf][j][vv];
      const f32x4* qv = reinterpret_cast<const f32x4*>(&qf[buf][j][0][dg * RD]);
      const f32x4* fv = reinterpret_cast<const f32x4*>(&qf[buf][j][1][dg * RD]);
      float po = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < RD / 4; ++i4) {
        const f32x4 q4 = qv[i4], f4 = fv[i4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[4 * i4 + e] = f4[e] * S[4 * i4 + e] + (1.0f - f4[e]) * v;
          po += S[4 * i4 + e] * q4[e];
        }
      }
      part[j][dg][vv] = po;
    }
    if (blk + 1 < nblk) stage(buf ^ 1);
    lds_barrier();     // the partial read-outs are complete
    for (int idx = threadIdx.x; idx < nt * 64; idx += NT) {
      const int j = idx >> 6, c = idx & 63;
      if (v0 + c < Dv) {
        float o = 0.f;
#pragma unroll
        for (int k = 0; k < HG_DG; ++k) o += part[j][k][c];
        out[((int64_t)q0 + blk * HG_TB + j) * os + (int64_t)h * Dv + v0 + c] = o;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < RD; ++i) {
    const int d = dg * RD + i;
    if (d < D && vok) Sp[(int64_t)d * Dv] = S[i];
  }
}

// Chunk-parallel form for long segments, around two runs of the kernel above over the chunks as segments of their own:
// hgrn2_decay: F[chunk][h D + d] = the product of the chunk's forget gates; hgrn2_combine: per segment, over its chunks
// in order, tmp[chunk] (the chunk's scan from zero) is replaced by the chunk's entry state and the running state
// becomes diag(F) state + local; the last one is the sequence's new state.
template <typename AT>
__global__ void hgrn2_decay_kernel(const AT* __restrict__ proj, int64_t ps, int f_off, const float* __restrict__ f_bias,
                                   const float* __restrict__ lower, int HD, const int* __restrict__ vseg,
                                   float* __restrict__ F) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= HD) return;
  const int ch = blockIdx.y;
  const int q0 = vseg[4 * ch], n = vseg[4 * ch + 1];
  const float lo = lower[c], fb = f_bias[c];
  float a = 1.f;
  for (int j0 = 0; j0 < n; j0 += 8) {   // eight rows' gates requested together
    float p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) p[j] = ldf(proj + ((int64_t)q0 + min(j0 + j, n - 1)) * ps + f_off + c);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j0 + j < n) a *= lo + (1.0f - lo) * sigmoidf(p[j] + fb);
  }
  F[(int64_t)ch * HD + c] = a;
}

__global__ void hgrn2_combine_kernel(const int* __restrict__ cs, const float* __restrict__ F, int HD, int Dv,
                                     float* __restrict__ tmp, float* __restrict__ state) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // (h, d, v) of the head matrices
  const int64_t n = (int64_t)HD * Dv;
  if (e >= n) return;
  const int r = blockIdx.y;
  const int first = cs[4 * r], cnt = cs[4 * r + 1], p0 = cs[4 * r + 2], slot = cs[4 * r + 3];
  const int hd = (int)(e / Dv);
  float S = p0 > 0 ? state[(int64_t)slot * n + e] : 0.f;
  for (int c = first; c < first + cnt; ++c) {
    const float L = tmp[(int64_t)c * n + e];
    tmp[(int64_t)c * n + e] = S;
    S = F[(int64_t)c * HD + hd] * S + L;
  }
  state[(int64_t)slot * n + e] = S;
}

// ---- attention inputs: rotation, head mix, paged store -------------------------------------------------------------------
// One workgroup per row of the fused projection [q (H D) | k (G D) | v (G Dv) | ...]. The row's q and k parts, the
// position's cos | sin row and the mix matrix are staged in LDS as fp32 in one batch of independent loads (a step of few
// rows pays one memory latency per row); pairs are rotated in place (a thread owns both members); keys leave for
// their page; the queries leave as they are, or with `talk` as q'[h][c D + i] = sum_r talk[h][c rep + r] q[c rep + r][i]
// (rep = H / G).
constexpr int MIX_REP = 32;   // query heads per key head whose values a lane keeps in registers for the head mix

template <typename AT>
__global__ __launch_bounds__(NT) void rope_kv_store_kernel(
    const AT* __restrict__ qkv, int64_t qs, int H, int G, int D, int Dv, const int64_t* __restrict__ positions,
    const float* __restrict__ cos_sin, int dims, bool pairs, const float* __restrict__ talk, AT* __restrict__ kc,
    AT* __restrict__ vt, const int64_t* __restrict__ slots, AT* __restrict__ q_out, int64_t qos) {
  extern __shared__ float lds[];   // [H D + G D] q | k, [dims] cos | sin, [H H] mix weights
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int Cq = H * D, Ck = G * D, Cv = G * Dv;
  const AT* row = qkv + t * qs;
  const int half = dims >> 1;
  float* qk = lds;
  float* cs = lds + Cq + Ck;
  float* tsh = cs + dims;
  const int64_t slot = slots[t];
  for (int i0 = 0; i0 < Cq + Ck; i0 += 8 * NT) {   // eight loads a thread in flight before the first LDS store
    float tmp[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = i0 + j * NT + threadIdx.x;
      tmp[j] = i < Cq + Ck ? ldf(row + i) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = i0 + j * NT + threadIdx.x;
      if (i < Cq + Ck) qk[i] = tmp[j];
    }
  }
  if (dims > 0) {
    const float* src = cos_sin + positions[t] * dims;
    for (int i = threadIdx.x; i < dims; i += NT) cs[i] = src[i];
  }
  if (talk != nullptr)
    for (int i = threadIdx.x; i < H * H; i += NT) tsh[i] = talk[i];
  if (slot >= 0) {
    AT* vd = vt + (slot / PAGE) * (int64_t)Cv * PAGE + (slot % PAGE);
#pragma unroll 4
    for (int i = threadIdx.x; i < Cv; i += NT) vd[(int64_t)i * PAGE] = row[Cq + Ck + i];
  }
  __syncthreads();
  // a wave per head (query heads, then key heads), lanes over its frequencies
  for (int hd = wave; hd < H + G; hd += NT / 64) {
    float* x = qk + hd * D;
    for (int f = lane; f < half; f += 64) {
      const int i0 = pairs ? 2 * f : f, i1 = pairs ? 2 * f + 1 : f + half;
      const float a = x[i0], b = x[i1], c = cs[f], sn = cs[half + f];
      x[i0] = a * c - b * sn;
      x[i1] = b * c + a * sn;
    }
  }
  __syncthreads();
  if (slot >= 0) {
    AT* kd = kc + slot * Ck;
    for (int i = threadIdx.x; i < Ck; i += NT) stf(kd + i, qk[Cq + i]);
  }
  if (talk == nullptr) {
    for (int i = threadIdx.x; i < Cq; i += NT) stf(q_out + t * qos + i, qk[i]);
    return;
  }
  const int rep = H / G;
  if (rep <= MIX_REP) {
    // a wave per (key head c, 64 of its dimensions): the rep query values of a lane's dimension stay in registers for
    // all H outputs; the weights are wave-uniform (broadcast) LDS reads, rep per output, all requested before the
    // multiply-adds
    const int wv = __builtin_amdgcn_readfirstlane(wave);
    const int nb = (D + 63) >> 6;
    for (int task = wv; task < G * nb; task += NT / 64) {
      const int c = task / nb, i = ((task - c * nb) << 6) + lane;
      // (loads at clamped, always valid addresses and a select afterwards: nothing between them that would make the
      // compiler wait for one LDS read before it issues the next)
      const int ic = min(i, D - 1);
      float qv[MIX_REP];
#pragma unroll
      for (int r = 0; r < MIX_REP; ++r) {
        const float v = qk[(c * rep + min(r, rep - 1)) * D + ic];
        qv[r] = (r < rep && i < D) ? v : 0.f;
      }
      for (int h = 0; h < H; ++h) {
        const float* tr = tsh + h * H + c * rep;
        float v0 = 0.f, v1 = 0.f;
#pragma unroll
        for (int r0 = 0; r0 < MIX_REP; r0 += 8) {
          if (r0 < rep) {   // (uniform) eight weights requested together; query values past rep are zero
            float wt[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) wt[j] = tr[min(r0 + j, rep - 1)];
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
              v0 += wt[j] * qv[r0 + j];
              v1 += wt[j + 1] * qv[r0 + j + 1];
            }
          }
        }
        if (i < D) stf(q_out + t * qos + ((int64_t)h * G + c) * D + i, v0 + v1);
      }
    }
    return;
  }
  for (int hc = wave; hc < H * G; hc += NT / 64) {
    const int h = hc / G, c = hc - h * G;
    const float* tr = tsh + h * H + c * rep;
    for (int i = lane; i < D; i += 64) {
      const float* qp = qk + (c * rep) * D + i;
      float v = 0.f;
      for (int r = 0; r < rep; ++r) v += tr[r] * qp[r * D];
      stf(q_out + t * qos + (int64_t)hc * D + i, v);
    }
  }
}

}  // namespace hp
}  // namespace kafka

using namespace kafka::hp;

#define DISPATCH_AT(f32, ...)             \
  if (f32) {                              \
    using AT = float;                     \
    __VA_ARGS__;                          \
  } else {                                \
    using AT = bf16;                      \
    __VA_ARGS__;                          \
  }

static inline int ew_grid(int64_t n) { return (int)std::min<int64_t>((n + 255) / 256, 65535 * 4); }

extern "C" {

hipError_t kafka_hy_act_norm(int f32, const void* x, int64_t xs, int c0, int n, const float* w, float eps, void* out,
                             int64_t os, int64_t T, int center, hipStream_t st) {
  if (T <= 0 || n <= 0) return hipSuccess;
  DISPATCH_AT(f32, {
    act_norm_kernel<AT><<<(unsigned)T, NT, 0, st>>>((const AT*)x, xs, c0, n, w, eps, (AT*)out, os, center != 0);
  });
  return hipGetLastError();
}

hipError_t kafka_hy_gate_mul(int f32, const void* a, int64_t as, const void* g, int64_t gs, int g_off, float scale,
                             void* out, int64_t os, int64_t T, int n, hipStream_t st) {
  if (T <= 0 || n <= 0) return hipSuccess;
  auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (!f32 && n % 8 == 0 && g_off % 8 == 0 && as % 8 == 0 && gs % 8 == 0 && os % 8 == 0 && al(a) && al(g) && al(out)) {
    gate_mul_vec8_kernel<<<ew_grid(T * (n / 8)), 256, 0, st>>>((const bf16*)a, as, (const bf16*)g, gs, g_off, scale,
                                                              (bf16*)out, os, T, n);
    return hipGetLastError();
  }
  DISPATCH_AT(f32, {
    gate_mul_kernel<AT><<<ew_grid(T * n), 256, 0, st>>>((const AT*)a, as, (const AT*)g, gs, g_off, scale, (AT*)out, os,
                                                        T, n);
  });
  return hipGetLastError();
}

int kafka_hy_mingru_chunk() { return MG_CH; }

hipError_t kafka_hy_mingru_scan(int f32, const void* proj, int64_t ps, const float* bias, const int* seg, int R,
                                float* state, void* out, int64_t os, int W, hipStream_t st) {
  if (R <= 0 || W <= 0) return hipSuccess;
  if (R > 65535) return hipErrorInvalidValue;
  const dim3 grid((W + 63) / 64, R);
  DISPATCH_AT(f32, {
    mingru_scan_kernel<AT><<<grid, 64, 0, st>>>((const AT*)proj, ps, bias, seg, state, (AT*)out, os, W);
  });
  return hipGetLastError();
}

// ab: fp32 [T, 2 W] scratch; ce: fp32 [R, nch, 2, W] scratch
hipError_t kafka_hy_mingru_scan_chunked(int f32, const void* proj, int64_t ps, const float* bias, const int* seg, int R,
                                        int nch, float* ab, float* ce, float* state, void* out, int64_t os, int64_t T,
                                        int W, hipStream_t st) {
  if (R <= 0 || W <= 0 || T <= 0) return hipSuccess;
  if (nch < 1 || ab == nullptr || ce == nullptr || nch > 65535 || R > 65535) return hipErrorInvalidValue;
  const dim3 gc((W + 63) / 64, nch, R), gk((W + 63) / 64, R);
  DISPATCH_AT(f32, {
    mingru_prep_kernel<AT><<<ew_grid(T * W), 256, 0, st>>>((const AT*)proj, ps, bias, ab, T, W);
    mingru_chunk_kernel<AT, 0><<<gc, 64, 0, st>>>(ab, (const AT*)proj, ps, seg, nch, ce, (AT*)out, os, W);
    mingru_carry_kernel<<<gk, 64, 0, st>>>(seg, nch, ce, state, W);
    mingru_chunk_kernel<AT, 1><<<gc, 64, 0, st>>>(ab, (const AT*)proj, ps, seg, nch, ce, (AT*)out, os, W);
  });
  return hipGetLastError();
}

int kafka_hy_hgrn2_max_d() { return HG_DG * 64; }

hipError_t kafka_hy_hgrn2_scan(int f32, const void* proj, int64_t ps, int q_off, int f_off, int v_off,
                               const float* f_bias, const float* lower, int H, int D, int Dv, const int* seg, int R,
                               float* S, float* out, int64_t os, hipStream_t st) {
  if (R <= 0) return hipSuccess;
  if (D > HG_DG * 64 || D < 1 || Dv < 1 || H < 1 || H > 65535 || R > 65535) return hipErrorInvalidValue;
  const dim3 grid((Dv + 63) / 64, H, R);
#define HG_LAUNCH(RD)                                                                                               \
  hgrn2_scan_kernel<AT, RD><<<grid, NT, 0, st>>>((const AT*)proj, ps, q_off, f_off, v_off, f_bias, lower, H, D, Dv, \
                                                 seg, S, out, os)
  DISPATCH_AT(f32, {
    if (D <= HG_DG * 16) HG_LAUNCH(16);
    else if (D <= HG_DG * 32) HG_LAUNCH(32);
    else HG_LAUNCH(64);
  });
#undef HG_LAUNCH
  return hipGetLastError();
}

hipError_t kafka_hy_hgrn2_decay(int f32, const void* proj, int64_t ps, int f_off, const float* f_bias,
                                const float* lower, int HD, const int* vseg, int n_chunks, float* F, hipStream_t st) {
  if (n_chunks <= 0 || HD <= 0) return hipSuccess;
  if (n_chunks > 65535) return hipErrorInvalidValue;
  const dim3 grid((HD + 63) / 64, n_chunks);
  DISPATCH_AT(f32, { hgrn2_decay_kernel<AT><<<grid, 64, 0, st>>>((const AT*)proj, ps, f_off, f_bias, lower, HD, vseg, F); });
  return hipGetLastError();
}

hipError_t kafka_hy_hgrn2_combine(const int* cs, int R, const float* F, int HD, int Dv, float* tmp, float* state,
                                  hipStream_t st) {
  if (R <= 0 || HD <= 0 || Dv <= 0) return hipSuccess;
  if (R > 65535) return hipErrorInvalidValue;
  const dim3 grid((unsigned)(((int64_t)HD * Dv + 255) / 256), R);
  hgrn2_combine_kernel<<<grid, 256, 0, st>>>(cs, F, HD, Dv, tmp, state);
  return hipGetLastError();
}

int kafka_hy_rope_store_max_q() { return 15360; }   // floats of LDS: H D + G D + rot dims (+ H H with a head mix)

hipError_t kafka_hy_rope_kv_store(int f32, const void* qkv, int64_t qs, int H, int G, int D, int Dv,
                                  const int64_t* positions, const float* cos_sin, int dims, int pairs,
                                  const float* talk, void* kc, void* vt, const int64_t* slots, void* q_out, int64_t qos,
                                  int64_t T, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (dims < 0 || dims % 2 || dims > D || (dims > 0 && cos_sin == nullptr) || G < 1 || H % G) return hipErrorInvalidValue;
  const int64_t fl = (int64_t)(H + G) * D + dims + (talk != nullptr ? H * H : 0);
  if (fl > kafka_hy_rope_store_max_q()) return hipErrorInvalidValue;
  const size_t lds = (size_t)fl * sizeof(float);
  DISPATCH_AT(f32, {
    rope_kv_store_kernel<AT><<<(unsigned)T, NT, lds, st>>>((const AT*)qkv, qs, H, G, D, Dv, positions, cos_sin, dims,
                                                           pairs != 0, talk, (AT*)kc, (AT*)vt, slots, (AT*)q_out, qos);
  });
  return hipGetLastError();
}

}  // extern "C"
