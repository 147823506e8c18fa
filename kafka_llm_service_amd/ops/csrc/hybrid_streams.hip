// Kernels for decoders with hyper-connected residual streams, windowed softmax attention with sinks and group-limited
// routing, for gfx950.
//
// Every kernel is built for bf16 and for fp32 activations; the residual streams and their mixing, norm statistics,
// rotation, attention scores and weights, router scores and the value mix are fp32 in both. Sizes are run-time values
// with no alignment assumptions.
//
//   stream_step         one pass over S residual streams [S][T][d] (fp32): the write of a sublayer's output (all
//                       streams at once from the old ones: x_r <- sum_s M[s][r] x_s + b_r y), the next sublayer's read
//                       u = sum_s a_s x_s with its RMS norm, and the plain sum - every part optional. One workgroup
//                       per row; a row's columns are loaded in one round, and its read values stay in registers
//                       between the statistics and the scaling.
//   swish_clamp_mul     g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit)
//   qk_norm_rope_store  RMS norm over the whole q and the whole k projection, rotation of dimension pairs (2i, 2i + 1),
//                       value mix with an earlier layer's values, paged key / transposed value store
//   window_attn         softmax attention with a sliding window and a sink logit; one wave per (row, head): lane = key
//                       for the scores (the query row broadcast from LDS), online softmax over 64-key blocks, then
//                       lane = value channel reading its channel's 16 consecutive tokens of a transposed page; a
//                       row's keys are visited in order, whatever the batch
//   window_attn_mfma    the same attention on the matrix cores (bf16): 32 (token, head) rows of one key/value head per
//                       workgroup, 128-key blocks, online softmax, key-range splits with a merge pass
//   moe_topk_grouped    softmax over all experts, choice among the best groups by corrected score, normalised weights
#include "common.h"

namespace kafka {
namespace hs {

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)(*p); }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }
// element i of a bf16 or fp32 array chosen at run time (uniform over the launch)
__device__ __forceinline__ float ldx(const void* p, bool f32, int64_t i) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : (float)reinterpret_cast<const bf16*>(p)[i];
}

constexpr int NT = 256;
constexpr int PAGE = 16;
constexpr float LOG2E = 1.4426950408889634f;

// Workgroup barrier for LDS hand-overs that leaves global loads (a prefetched next block) in flight: __syncthreads()
// would drain them as well. This wave's LDS reads and writes are complete (lgkmcnt 0) before it arrives.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- residual streams ----------------------------------------------------------------------------------------------
constexpr int SMAX = 16;   // streams
// columns of a row a thread keeps in registers (all S streams of each): rows up to NT * stream_nv(S) wide are loaded in
// one round of independent loads, written once, and their read values wait in registers for the row's mean square;
// wider rows walk the rest column by column and recompute the read values from the streams just written
__host__ __device__ constexpr int stream_nv(int S) { return S <= 4 ? 16 : S <= 8 ? 8 : 4; }

template <int S>
__global__ __launch_bounds__(NT) void stream_step_kernel(float* __restrict__ xs, int64_t s_stride, int64_t t_stride,
                                                         const void* __restrict__ y, int64_t ys, bool y_f32,
                                                         const void* __restrict__ y2, int64_t y2s, bool y2_f32,
                                                         const float* __restrict__ row_scale,
                                                         const float* __restrict__ mix, const float* __restrict__ wr,
                                                         const float* __restrict__ rd, const float* __restrict__ nw,
                                                         float eps, void* __restrict__ out, int64_t os, bool out_f32,
                                                         float* __restrict__ total, int64_t ts, int d, bool center) {
  constexpr int NV = stream_nv(S);
  __shared__ float red[NT / 64];
  __shared__ float cM[SMAX * SMAX], cb[SMAX], ca[SMAX];
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < S * S; i += NT)
    if (mix != nullptr) cM[i] = mix[i];
  if (threadIdx.x < S) {
    if (wr != nullptr) cb[threadIdx.x] = wr[threadIdx.x];
    if (rd != nullptr) ca[threadIdx.x] = rd[threadIdx.x];
  }
  __syncthreads();
  float* xr = xs + t * t_stride;
  const float rs2 = y2 != nullptr ? row_scale[t] : 0.f;
  // new stream values of one column from the old ones and the sublayer's output
  auto write = [&](float (&x)[S], float yv) {
    float nx[S];
#pragma unroll
    for (int r = 0; r < S; ++r) {
      float v = cb[r] * yv;
#pragma unroll
      for (int s = 0; s < S; ++s) v += cM[s * S + r] * x[s];
      nx[r] = v;
    }
#pragma unroll
    for (int s = 0; s < S; ++s) x[s] = nx[s];
  };
  auto read = [&](const float (&x)[S]) {
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < S; ++s) u += ca[s] * x[s];
    return u;
  };
  float xv[NV][S], yv[NV];
  float acc = 0.f, accs = 0.f;   // sum of squares and plain sum of the read values
  // the register part: every load of the row's first NT * NV columns is issued before anything is stored
#pragma unroll
  for (int it = 0; it < NV; ++it) {
    const int i = threadIdx.x + it * NT;
    yv[it] = 0.f;
    if (i < d) {
#pragma unroll
      for (int s = 0; s < S; ++s) xv[it][s] = xr[s * s_stride + i];
      if (mix != nullptr) {
        yv[it] = ldx(y, y_f32, t * ys + i);
        if (y2 != nullptr) yv[it] += rs2 * ldx(y2, y2_f32, t * y2s + i);
      }
    }
  }
#pragma unroll
  for (int it = 0; it < NV; ++it) {
    const int i = threadIdx.x + it * NT;
    if (i < d) {
      if (mix != nullptr) {
        write(xv[it], yv[it]);
#pragma unroll
        for (int s = 0; s < S; ++s) xr[s * s_stride + i] = xv[it][s];
      }
      if (total != nullptr) {
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < S; ++s) v += xv[it][s];
        total[t * ts + i] = v;
      }
      if (rd != nullptr) {
        const float u = read(xv[it]);
        acc += u * u;
        accs += u;
        yv[it] = u;  // (the sublayer output is used up: its register keeps the read value)
      }
    }
  }
  for (int i = threadIdx.x + NV * NT; i < d; i += NT) {
    float x[S];
#pragma unroll
    for (int s = 0; s < S; ++s) x[s] = xr[s * s_stride + i];
    if (mix != nullptr) {
      float v = ldx(y, y_f32, t * ys + i);
      if (y2 != nullptr) v += rs2 * ldx(y2, y2_f32, t * y2s + i);
      write(x, v);
#pragma unroll
      for (int s = 0; s < S; ++s) xr[s * s_stride + i] = x[s];
    }
    if (total != nullptr) {
      float v = 0.f;
#pragma unroll
      for (int s = 0; s < S; ++s) v += x[s];
      total[t * ts + i] = v;
    }
    if (rd != nullptr) {
      const float u = read(x);
      acc += u * u;
      accs += u;
    }
  }
  if (rd == nullptr) return;
  // a centred norm takes the row's mean off first and measures the deviations in a second pass over the read values
  float mean = 0.f;
  if (center) {
    mean = block_sum<NT>(accs, red) / (float)d;
    acc = 0.f;
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int i = threadIdx.x + it * NT;
      if (i < d) acc += (yv[it] - mean) * (yv[it] - mean);
    }
    for (int i = threadIdx.x + NV * NT; i < d; i += NT) {
      float x[S];
#pragma unroll
      for (int s = 0; s < S; ++s) x[s] = xr[s * s_stride + i];
      const float u = read(x) - mean;
      acc += u * u;
    }
  }
  const float rs = 1.0f / sqrtf(block_sum<NT>(acc, red) / (float)d + eps);
  auto store = [&](int i, float u) {
    const float v = (u - mean) * rs * nw[i];
    if (out_f32) reinterpret_cast<float*>(out)[t * os + i] = v;
    else reinterpret_cast<bf16*>(out)[t * os + i] = (bf16)v;
  };
#pragma unroll
  for (int it = 0; it < NV; ++it) {
    const int i = threadIdx.x + it * NT;
    if (i < d) store(i, yv[it]);
  }
  for (int i = threadIdx.x + NV * NT; i < d; i += NT) {  // (this thread's own writes of the first pass)
    float x[S];
#pragma unroll
    for (int s = 0; s < S; ++s) x[s] = xr[s * s_stride + i];
    store(i, read(x));
  }
}

template <typename AT>
__global__ void swish_clamp_mul_kernel(const AT* __restrict__ gu, int64_t gs, AT* __restrict__ out, int64_t os, int64_t T,
                                       int F, float limit, float alpha) {
  const int64_t n = T * F;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / F;
    const int f = (int)(i - t * F);
    const float g = fminf(ldf(gu + t * gs + f), limit);
    const float u = fminf(fmaxf(ldf(gu + t * gs + F + f), -limit), limit);
    stf(out + t * os + f, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
  }
}

// the same on bf16 rows whose sizes, strides and bases are multiples of 8 elements: 8 gate and 8 up values per thread step
__global__ void swish_clamp_mul_vec8_kernel(const bf16* __restrict__ gu, int64_t gs, bf16* __restrict__ out, int64_t os,
                                            int64_t T, int F, float limit, float alpha) {
  const int F8 = F >> 3;
  const int64_t n = T * F8;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / F8;
    const int f = (int)(i - t * F8) << 3;
    const bf16x8 gv = load_bf16x8(gu + t * gs + f), uv = load_bf16x8(gu + t * gs + F + f);
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float g = fminf((float)gv[j], limit);
      const float u = fminf(fmaxf((float)uv[j], -limit), limit);
      o[j] = (bf16)(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
    }
    store_bf16x8(out + t * os + f, o);
  }
}

// ---- attention inputs ------------------------------------------------------------------------------------------------
// one workgroup per row of the fused projection [q (H D) | k (G D) | v (G Dv)]
template <typename AT>
__global__ __launch_bounds__(NT) void qk_norm_rope_store_kernel(
    const AT* __restrict__ qkv, int64_t qs, int H, int G, int D, int Dv, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps, const int64_t* __restrict__ positions, const float* __restrict__ cos_sin,
    int dims, const AT* __restrict__ vf, int64_t vfs, int vf_off, float lam, AT* __restrict__ kc, AT* __restrict__ vt,
    const int64_t* __restrict__ slots, AT* __restrict__ q_out, int64_t qos) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int Cq = H * D, Ck = G * D, Cv = G * Dv;
  const AT* row = qkv + t * qs;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < Cq; i += NT) {
    const float v = ldf(row + i);
    sq += v * v;
  }
  for (int i = threadIdx.x; i < Ck; i += NT) {
    const float v = ldf(row + Cq + i);
    sk += v * v;
  }
  const float rq = 1.0f / sqrtf(block_sum<NT>(sq, red) / (float)Cq + eps);
  const float rk = 1.0f / sqrtf(block_sum<NT>(sk, red) / (float)Ck + eps);
  const int half = dims >> 1;
  const float* cs = dims > 0 ? cos_sin + positions[t] * dims : nullptr;
  const int64_t slot = slots[t];
  // element i of a normed projection, rotated with its pair partner when it lies in a head's first `dims` dimensions
  auto elem = [&](const AT* src, const float* w, float r, int i) {
    const float a = ldf(src + i) * r * w[i];
    const int dh = i % D;
    if (dh >= dims) return a;
    const int ip = (dh & 1) ? i - 1 : i + 1;  // the pair partner within the head
    const float b = ldf(src + ip) * r * w[ip];
    const float c = cs[dh >> 1], s = cs[half + (dh >> 1)];
    return (dh & 1) ? a * c + b * s : a * c - b * s;
  };
  for (int i = threadIdx.x; i < Cq; i += NT) stf(q_out + t * qos + i, elem(row, qw, rq, i));
  if (slot < 0) return;
  AT* kd = kc + slot * Ck;
  for (int i = threadIdx.x; i < Ck; i += NT) stf(kd + i, elem(row + Cq, kw, rk, i));
  AT* vd = vt + (slot / PAGE) * (int64_t)Cv * PAGE + (slot % PAGE);
  for (int i = threadIdx.x; i < Cv; i += NT) {
    float v = ldf(row + Cq + Ck + i);
    if (vf != nullptr) v = (1.0f - lam) * v + lam * ldf(vf + t * vfs + vf_off + i);
    stf(vd + (int64_t)i * PAGE, v);
  }
}

// ---- windowed softmax attention with a sink -----------------------------------------------------------------------
constexpr int WA_MAXD = 1024;  // query / key size (the query row sits in LDS as fp32)
constexpr int WA_NV = 8;      // value size up to 64 * WA_NV

template <typename AT>
__global__ __launch_bounds__(NT) void window_attn_kernel(const AT* __restrict__ q, int64_t qs,
                                                         const AT* __restrict__ kc, const AT* __restrict__ vt,
                                                         const int* __restrict__ bt, int bt_stride,
                                                         const int* __restrict__ tok_seg,
                                                         const int64_t* __restrict__ positions, int H, int G, int D,
                                                         int Dv, int Ck, int kstep, float scale_log2e, int window,
                                                         const float* __restrict__ sink, AT* __restrict__ out,
                                                         int64_t os, int64_t pairs) {
  // D: size of a query row and of the key it meets; key/value head g's key starts at column g * kstep of a key row of
  // Ck columns (kstep = D: one key head per key/value head; kstep = 0, D = Ck: every query row meets the whole key row)
  __shared__ float qsh[NT / 64][WA_MAXD];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t pair = (int64_t)blockIdx.x * (NT / 64) + wave;
  if (pair >= pairs) return;  // whole waves leave; nothing below synchronises across waves
  const int64_t t = pair / H;
  const int h = (int)(pair - t * H);
  const int g = h / (H / G);
  const int64_t p = positions[t];
  const int* pages = bt + (int64_t)tok_seg[t] * bt_stride;
  float* qw = qsh[wave];
  for (int i = lane; i < D; i += 64) qw[i] = ldf(q + t * qs + (int64_t)h * D + i) * scale_log2e;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int Cv = G * Dv;
  float acc[WA_NV];
#pragma unroll
  for (int i = 0; i < WA_NV; ++i) acc[i] = 0.f;
  // the sink is a term of the denominator without a value: the running maximum and sum start from it
  float m = -INFINITY, l = 0.f;
  if (sink != nullptr) {
    m = sink[h] * LOG2E;
    l = 1.f;
  }
  const int64_t lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;  // first visible key
  for (int64_t j0 = lo & ~(int64_t)(PAGE - 1); j0 <= p; j0 += 64) {
    const int64_t j = j0 + lane;
    float s = -INFINITY;
    if (j <= p && j >= lo) {
      const AT* kr = kc + ((int64_t)pages[j / PAGE] * PAGE + (j % PAGE)) * Ck + (int64_t)g * kstep;
      float dot = 0.f;
      for (int i = 0; i < D; ++i) dot += qw[i] * ldf(kr + i);
      s = dot;
    }
    const float mn = fmaxf(m, wave_max(s));  // finite: the block holds a visible key (j0 <= p and j0 + 63 >= lo)
    const float corr = fast_exp2(m - mn);    // 0 while m is -inf
    const float w = fast_exp2(s - mn);       // 0 for masked keys
    l = l * corr + wave_sum(w);
    m = mn;
    const int nk = (int)((p - j0 + 1 < 64) ? (p - j0 + 1) : 64);  // keys of this block up to the row's own
#pragma unroll
    for (int i = 0; i < WA_NV; ++i) acc[i] *= corr;
    for (int pg = 0; pg * PAGE < nk; ++pg) {
      const int64_t page = pages[(j0 >> 4) + pg];
      const int ne = (nk - pg * PAGE < PAGE) ? nk - pg * PAGE : PAGE;
      float wk[PAGE];
#pragma unroll
      for (int e = 0; e < PAGE; ++e) wk[e] = __shfl(w, pg * PAGE + e, 64);
#pragma unroll
      for (int i = 0; i < WA_NV; ++i) {
        const int v = lane + 64 * i;
        if (v < Dv) {
          const AT* vp = vt + (page * Cv + (int64_t)g * Dv + v) * PAGE;
          float a = acc[i];
#pragma unroll
          for (int e = 0; e < PAGE; ++e)
            if (e < ne) a += wk[e] * ldf(vp + e);
          acc[i] = a;
        }
      }
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < WA_NV; ++i) {
    const int v = lane + 64 * i;
    if (v < Dv) stf(out + t * os + (int64_t)h * Dv + v, acc[i] * inv);
  }
}

// ---- windowed softmax attention on the matrix cores (bf16) --------------------------------------------------------
// One workgroup (4 waves) per (tile, key/value head): a tile is 32 query rows = (token, query head of this key/value
// head) pairs of consecutive tokens of one segment (floor(32 / rep) tokens, rep = H / G query heads per key/value
// head). Keys go by in blocks of 128, from the block that holds the first key the tile's first row sees:
//   scores   wave w takes keys 32 w .. 32 w + 31 of the block: S = Q K^T as D / 16 MFMA steps (32x32x16), the Q tile
//            read from LDS, the key rows straight from the paged cache (lane = key, 16 bytes per step), the next
//            block's rows requested before this block's softmax;
//   softmax  keys ahead of the row or behind its window count as -inf; row maxima within the wave by lane exchange
//            and across the four waves through LDS; P = 2^(S - m) goes to LDS as bf16; the row sums stay per lane
//            and are combined once at the end;
//   values   wave w owns output columns [32 TW w, 32 TW (w + 1)): O += P V with V read from the page-wise transposed
//            values (lane = column, 8 consecutive keys = 16 bytes), one page per MFMA step.
// Scores, maxima, sums and accumulators are fp32. The sink joins the denominator once, at the end. With
// gridDim.z > 1 the tile's key blocks are dealt to gridDim.z workgroups in contiguous ranges; each leaves its
// unnormalised accumulators in po [z][T][H Dv] and (row maximum, row sum) in pml [z][T][H][2] for window_merge.
// Needs 16-token pages, D % 16 == 0, at most 32 query heads per key/value head.
constexpr int WM_ROWS = 32;

template <int TW, int NKSC>
__global__ __launch_bounds__(256) void window_attn_mfma_kernel(
    const bf16* __restrict__ q, int64_t qs, const bf16* __restrict__ kc, const bf16* __restrict__ vt,
    const int* __restrict__ bt, int bt_stride, const int* __restrict__ items, const int64_t* __restrict__ positions,
    int H, int G, int D, int Dv, int Ck, int kstep, float scale_log2e, int window, const float* __restrict__ sink,
    bf16* __restrict__ out, int64_t os, float* __restrict__ po, float* __restrict__ pml, int64_t T) {
  // (D, Ck, kstep as in window_attn_kernel: kstep = 0 and D = Ck when every query row meets the whole key row)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int nks = D >> 4, qstride = D + 8;
  bf16* Qs = reinterpret_cast<bf16*>(smem);                       // [32][D + 8]
  bf16* Ps = Qs + WM_ROWS * qstride;                              // [32][128 + 8]
  float* mloc = reinterpret_cast<float*>(Ps + WM_ROWS * 136);     // [4][32]
  int* prow_s = reinterpret_cast<int*>(mloc + 4 * WM_ROWS);       // [32]
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, lr = lane & 31, lh = lane >> 5;
  const int t0 = items[4 * blockIdx.x], ntok = items[4 * blockIdx.x + 1], sg = items[4 * blockIdx.x + 2];
  const int g = blockIdx.y, rep = H / G;
  const int nrows = ntok * rep;
  for (int i = threadIdx.x; i < WM_ROWS * (D >> 3); i += 256) {
    const int r = i / (D >> 3), d0 = (i - r * (D >> 3)) << 3;
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (r < nrows) v = load_bf16x8(q + (int64_t)(t0 + r / rep) * qs + (int64_t)(g * rep + r % rep) * D + d0);
    store_bf16x8(Qs + r * qstride + d0, v);
  }
  // a row beyond the tile sees no key
  if (threadIdx.x < WM_ROWS) prow_s[threadIdx.x] = threadIdx.x < nrows ? (int)positions[t0 + threadIdx.x / rep] : -1;
  const int maxpos = (int)positions[t0 + ntok - 1];
  __syncthreads();
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
  const int Cv = G * Dv;
  const int nblocks = (maxpos >> 7) + 1;
  const int kbmin = window > 0 ? max(0, (int)positions[t0] - window + 1) >> 7 : 0;
  const bf16* qrow = Qs + lr * qstride + 8 * lh;
  bf16x8 kf[NKSC];
  auto fetch_keys = [&](int kb) {
    const int kcix = min(kb * 128 + 32 * w + lr, maxpos);  // past the tile's last position: a valid row, masked below
    const bf16* krow = kc + ((int64_t)btr[kcix >> 4] * PAGE + (kcix & 15)) * Ck + (int64_t)g * kstep + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < NKSC; ++ks)
      if (ks < nks) kf[ks] = load_bf16x8(krow + 16 * ks);
  };
  const int nsplit = gridDim.z;
  const int bps = (nblocks - kbmin + nsplit - 1) / nsplit;
  const int kb0 = kbmin + blockIdx.z * bps, kb1 = min(nblocks, kb0 + bps);
  if (kb0 < kb1 && kb0 * 128 + 32 * w <= maxpos) fetch_keys(kb0);
  for (int kb = kb0; kb < kb1; ++kb) {
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
      // first block: m = -inf -> corr 0. A range may lie wholly outside a row's window: then mn is still -inf and
      // the row stays empty (the guards keep inf - inf out)
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
        const bf16* vp = vt + ((int64_t)btr[kb * 8 + k0 + kk] * Cv + (int64_t)g * Dv) * PAGE + 8 * lh;
#pragma unroll
        for (int tw = 0; tw < TW; ++tw) {
          const int col = (w * TW + tw) * 32 + lr;
          bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
          vf[kk][tw] = col < Dv ? load_bf16x8(vp + (int64_t)col * PAGE) : z;
        }
      }
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        if ((kb * 8 + k0 + kk) * 16 > maxpos) break;
        const bf16x8 a = load_bf16x8(Ps + lr * 136 + 16 * (k0 + kk) + 8 * lh);
#pragma unroll
        for (int tw = 0; tw < TW; ++tw)
          if ((w * TW + tw) * 32 < Dv) O[tw] = mfma32(a, vf[kk][tw], O[tw]);
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
    const int64_t t = t0 + r / rep;
    const int h = g * rep + r % rep;
    if (nsplit == 1) {
      if (sink != nullptr) l += fast_exp2(sink[h] * LOG2E - m[i]);
      const float inv = 1.0f / l;
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) {
        const int col = (w * TW + tw) * 32 + lr;
        if (col < Dv) out[t * os + (int64_t)h * Dv + col] = (bf16)(O[tw][i] * inv);
      }
    } else {
      const int64_t row = ((int64_t)blockIdx.z * T + t) * H + h;
      if (w == 0 && lr == 0) {
        pml[2 * row] = m[i];
        pml[2 * row + 1] = l;
      }
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) {
        const int col = (w * TW + tw) * 32 + lr;
        if (col < Dv) po[row * Dv + col] = O[tw][i];
      }
    }
  }
}

// out[t][h] = sum_z 2^(m_z - m) O_z / (sum_z 2^(m_z - m) l_z + 2^(sink_h - m)) over the key-range splits
__global__ void window_merge_kernel(const float* __restrict__ po, const float* __restrict__ pml, int nsplit, int64_t T,
                                    int H, int Dv, const float* __restrict__ sink, bf16* __restrict__ out, int64_t os) {
  const int64_t th = blockIdx.x;  // t * H + h
  const int64_t t = th / H;
  const int h = (int)(th - t * H);
  const int64_t zs = T * H;
  float mx = -INFINITY;
  for (int z = 0; z < nsplit; ++z) mx = fmaxf(mx, pml[2 * (z * zs + th)]);
  float den = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float mz = pml[2 * (z * zs + th)];
    if (mz != -INFINITY) den += fast_exp2(mz - mx) * pml[2 * (z * zs + th) + 1];
  }
  if (sink != nullptr) den += fast_exp2(sink[h] * LOG2E - mx);
  const float inv = 1.0f / den;
  for (int d = threadIdx.x; d < Dv; d += blockDim.x) {
    float a = 0.f;
    for (int z = 0; z < nsplit; ++z) {
      const float mz = pml[2 * (z * zs + th)];
      if (mz != -INFINITY) a += fast_exp2(mz - mx) * po[(z * zs + th) * Dv + d];
    }
    out[t * os + (int64_t)h * Dv + d] = (bf16)(a * inv);
  }
}

// ---- group-limited router ------------------------------------------------------------------------------------------
constexpr int GR_MAXE = 512;  // experts (8 per lane)
constexpr int GR_MAXK = 16;
constexpr int GR_MAXG = 64;   // groups (one per lane)

// one wave per row of fp32 logits [T, >= E]: s = softmax over the E experts; c = s + correction; the `keep` groups
// (of `groups` equal runs of neighbouring experts) with the largest max c stay, the others' c count as -inf; the k
// largest c are chosen (ties: the lower index); weights = s of the chosen / (their sum + eps). With `gate` the
// logit in column E goes through a sigmoid.
__global__ __launch_bounds__(NT) void moe_topk_grouped_kernel(const float* __restrict__ logits, int64_t ls, int E,
                                                              int k, const float* __restrict__ corr, int groups,
                                                              int keep, float eps, float* __restrict__ tw,
                                                              int* __restrict__ te, float* __restrict__ gate,
                                                              int64_t T) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * (NT / 64) + wave;
  if (t >= T) return;
  constexpr int PL = GR_MAXE / 64;
  float sc[PL], c[PL];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < PL; ++i) {
    const int e = lane + 64 * i;
    sc[i] = e < E ? logits[t * ls + e] : -INFINITY;
    mx = fmaxf(mx, sc[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < PL; ++i) {
    sc[i] = lane + 64 * i < E ? expf(sc[i] - mx) : 0.f;
    sum += sc[i];
  }
  sum = wave_sum(sum);
  const int gsz = E / groups;
#pragma unroll
  for (int i = 0; i < PL; ++i) {
    const int e = lane + 64 * i;
    sc[i] = sc[i] / sum;
    c[i] = e < E ? sc[i] + corr[e] : -INFINITY;
  }
  if (keep < groups) {
    // lane g holds group g's score
    float gs = -INFINITY;
    for (int g = 0; g < groups; ++g) {
      float v = -INFINITY;
#pragma unroll
      for (int i = 0; i < PL; ++i) {
        const int e = lane + 64 * i;
        if (e < E && e / gsz == g) v = fmaxf(v, c[i]);
      }
      v = wave_max(v);
      if (lane == g) gs = v;
    }
    unsigned long long kept = 0ull;
    for (int j = 0; j < keep; ++j) {
      float bv = gs;
      int bi = lane < groups ? lane : 0x7fffffff;
      if (lane >= groups || ((kept >> lane) & 1ull)) { bv = -INFINITY; bi = 0x7fffffff; }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
      }
      kept |= 1ull << bi;
    }
#pragma unroll
    for (int i = 0; i < PL; ++i) {
      const int e = lane + 64 * i;
      if (e < E && !((kept >> (e / gsz)) & 1ull)) c[i] = -INFINITY;
    }
  }
  float val[GR_MAXK];
  float wsum = 0.f;
  unsigned taken = 0u;  // this lane's experts already chosen (bit i: expert lane + 64 i)
  for (int j = 0; j < k; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < PL; ++i) {
      const int e = lane + 64 * i;
      if (e < E && !((taken >> i) & 1u) && (bi == 0x7fffffff || c[i] > bv)) { bv = c[i]; bi = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
    }
    float mine = 0.f;
#pragma unroll
    for (int i = 0; i < PL; ++i)
      if (bi == lane + 64 * i) {
        taken |= 1u << i;
        mine = sc[i];
      }
    const float sv = __shfl(mine, bi & 63, 64);
    if (j < GR_MAXK) val[j] = sv;
    wsum += sv;
    if (lane == 0) te[t * k + j] = bi;
  }
  if (lane == 0) {
    const float inv = 1.0f / (wsum + eps);
    for (int j = 0; j < k; ++j) tw[t * k + j] = val[j] * inv;
    if (gate != nullptr) gate[t] = 1.0f / (1.0f + expf(-logits[t * ls + E]));
  }
}

static inline int ew_grid(int64_t n) { return (int)std::min<int64_t>((n + 255) / 256, 65535 * 4); }

}  // namespace hs
}  // namespace kafka

using namespace kafka::hs;

#define DISPATCH_AT(f32, ...)             \
  if (f32) {                              \
    using AT = float;                     \
    __VA_ARGS__;                          \
  } else {                                \
    using AT = bf16;                      \
    __VA_ARGS__;                          \
  }

extern "C" {

int kafka_hy_stream_max() { return SMAX; }

hipError_t kafka_hy_stream_step(float* xs, int64_t s_stride, int64_t t_stride, int S, const void* y, int64_t ys,
                                int y_f32, const void* y2, int64_t y2s, int y2_f32, const float* row_scale,
                                const float* mix, const float* wr, const float* rd, const float* nw, float eps,
                                void* out, int64_t os, int out_f32, float* total, int64_t ts, int64_t T, int d,
                                int center, hipStream_t st) {
  if (T <= 0 || d <= 0) return hipSuccess;
  if (S < 1 || S > SMAX) return hipErrorInvalidValue;
  auto a = [&](auto k) {
    k<<<(unsigned)T, NT, 0, st>>>(xs, s_stride, t_stride, y, ys, y_f32 != 0, y2, y2s, y2_f32 != 0, row_scale, mix, wr,
                                  rd, nw, eps, out, os, out_f32 != 0, total, ts, d, center != 0);
  };
  switch (S) {
    case 1: a(stream_step_kernel<1>); break;
    case 2: a(stream_step_kernel<2>); break;
    case 3: a(stream_step_kernel<3>); break;
    case 4: a(stream_step_kernel<4>); break;
    case 5: a(stream_step_kernel<5>); break;
    case 6: a(stream_step_kernel<6>); break;
    case 7: a(stream_step_kernel<7>); break;
    case 8: a(stream_step_kernel<8>); break;
    case 9: a(stream_step_kernel<9>); break;
    case 10: a(stream_step_kernel<10>); break;
    case 11: a(stream_step_kernel<11>); break;
    case 12: a(stream_step_kernel<12>); break;
    case 13: a(stream_step_kernel<13>); break;
    case 14: a(stream_step_kernel<14>); break;
    case 15: a(stream_step_kernel<15>); break;
    default: a(stream_step_kernel<16>); break;
  }
  return hipGetLastError();
}

hipError_t kafka_hy_swish_clamp_mul(int f32, const void* gu, int64_t gs, void* out, int64_t os, int64_t T, int F,
                                    float limit, float alpha, hipStream_t st) {
  if (T <= 0 || F <= 0) return hipSuccess;
  if (!f32 && F % 8 == 0 && gs % 8 == 0 && os % 8 == 0 && (reinterpret_cast<uintptr_t>(gu) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    swish_clamp_mul_vec8_kernel<<<ew_grid(T * (F / 8)), 256, 0, st>>>((const bf16*)gu, gs, (bf16*)out, os, T, F, limit,
                                                                      alpha);
    return hipGetLastError();
  }
  DISPATCH_AT(f32, {
    swish_clamp_mul_kernel<AT><<<ew_grid(T * F), 256, 0, st>>>((const AT*)gu, gs, (AT*)out, os, T, F, limit, alpha);
  });
  return hipGetLastError();
}

hipError_t kafka_hy_qk_norm_rope_store(int f32, const void* qkv, int64_t qs, int H, int G, int D, int Dv,
                                       const float* qw, const float* kw, float eps, const int64_t* positions,
                                       const float* cos_sin, int dims, const void* vf, int64_t vfs, int vf_off,
                                       float lam, void* kc, void* vt, const int64_t* slots, void* q_out, int64_t qos,
                                       int64_t T, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (dims < 0 || dims % 2 || dims > D || (dims > 0 && cos_sin == nullptr)) return hipErrorInvalidValue;
  DISPATCH_AT(f32, {
    qk_norm_rope_store_kernel<AT><<<(unsigned)T, NT, 0, st>>>((const AT*)qkv, qs, H, G, D, Dv, qw, kw, eps, positions,
                                                              cos_sin, dims, (const AT*)vf, vfs, vf_off, lam, (AT*)kc,
                                                              (AT*)vt, slots, (AT*)q_out, qos);
  });
  return hipGetLastError();
}

int kafka_hy_window_attn_max_d() { return WA_MAXD; }
int kafka_hy_window_attn_max_dv() { return 64 * WA_NV; }

hipError_t kafka_hy_window_attn(int f32, const void* q, int64_t qs, const void* kc, const void* vt, const int* bt,
                                int bt_stride, const int* tok_seg, const int64_t* positions, int H, int G, int D,
                                int Dv, float scale, int window, const float* sink, void* out, int64_t os, int64_t T,
                                int shared_keys, hipStream_t st) {
  // shared_keys: D is the whole key row's size and every query row meets all G key heads of a token at once
  if (T <= 0) return hipSuccess;
  if (D > WA_MAXD || Dv > 64 * WA_NV || G < 1 || H % G || window < 0) return hipErrorInvalidValue;
  const int64_t pairs = T * H;
  const int grid = (int)((pairs + NT / 64 - 1) / (NT / 64));
  const int Ck = shared_keys ? D : G * D, kstep = shared_keys ? 0 : D;
  DISPATCH_AT(f32, {
    window_attn_kernel<AT><<<grid, NT, 0, st>>>((const AT*)q, qs, (const AT*)kc, (const AT*)vt, bt, bt_stride, tok_seg,
                                                positions, H, G, D, Dv, Ck, kstep, scale * LOG2E, window, sink,
                                                (AT*)out, os, pairs);
  });
  return hipGetLastError();
}

// bf16 shapes the matrix-core kernel takes (else the per-wave kernel above runs)
int kafka_hy_window_attn_mfma_ok(int page, int D, int Dv, int rep) {
  return page == PAGE && D >= 16 && D % 16 == 0 && D <= 256 && Dv >= 1 && Dv <= 256 && rep >= 1 && rep <= WM_ROWS;
}

hipError_t kafka_hy_window_attn_mfma(const void* q, int64_t qs, const void* kc, const void* vt, const int* bt,
                                     int bt_stride, const int* items, int n_items, const int64_t* positions, int H,
                                     int G, int D, int Dv, float scale, int window, const float* sink, void* out,
                                     int64_t os, int nsplit, float* po, float* pml, int64_t T, int shared_keys,
                                     hipStream_t st) {
  if (n_items <= 0) return hipSuccess;
  const int Ck = shared_keys ? D : G * D, kstep = shared_keys ? 0 : D;
  if (G < 1 || H % G || window < 0 || !kafka_hy_window_attn_mfma_ok(PAGE, D, Dv, H / G)) return hipErrorInvalidValue;
  if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && (po == nullptr || pml == nullptr))) return hipErrorInvalidValue;
  const size_t lds = (size_t)WM_ROWS * (D + 8) * 2 + WM_ROWS * 136 * 2 + 5 * WM_ROWS * 4;
  const dim3 grid((unsigned)n_items, (unsigned)G, (unsigned)nsplit);
  auto a = [&](auto k) {
    k<<<grid, 256, lds, st>>>((const bf16*)q, qs, (const bf16*)kc, (const bf16*)vt, bt, bt_stride, items, positions, H,
                              G, D, Dv, Ck, kstep, scale * LOG2E, window, sink, (bf16*)out, os, po, pml, T);
  };
  const int nks = D / 16, tw = ((Dv + 31) / 32 + 3) / 4;
  if (tw == 1 && nks <= 4) a(window_attn_mfma_kernel<1, 4>);
  else if (tw == 1 && nks <= 8) a(window_attn_mfma_kernel<1, 8>);
  else if (tw == 1) a(window_attn_mfma_kernel<1, 16>);
  else if (nks <= 8) a(window_attn_mfma_kernel<2, 8>);
  else a(window_attn_mfma_kernel<2, 16>);
  if (nsplit > 1)
    window_merge_kernel<<<(unsigned)(T * H), 64, 0, st>>>(po, pml, nsplit, T, H, Dv, sink, (bf16*)out, os);
  return hipGetLastError();
}

int kafka_hy_grouped_router_max_e() { return GR_MAXE; }
int kafka_hy_grouped_router_max_k() { return GR_MAXK; }
int kafka_hy_grouped_router_max_g() { return GR_MAXG; }

hipError_t kafka_hy_moe_topk_grouped(const float* logits, int64_t ls, int E, int k, const float* corr, int groups,
                                     int keep, float eps, float* tw, int* te, float* gate, int64_t T, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (E > GR_MAXE || k > GR_MAXK || k < 1 || groups < 1 || groups > GR_MAXG || E % groups || keep < 1 ||
      keep > groups || k > keep * (E / groups))
    return hipErrorInvalidValue;
  const int grid = (int)((T + NT / 64 - 1) / (NT / 64));
  moe_topk_grouped_kernel<<<grid, NT, 0, st>>>(logits, ls, E, k, corr, groups, keep, eps, tw, te, gate, T);
  return hipGetLastError();
}

}  // extern "C"
