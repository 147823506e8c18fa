// Kernels of the gated mixers of the hybrid decoder family for gfx950: RMS norm of the fp32 stream, paged key / value
// store, sigmoid attention (no softmax), the real-gated linear recurrence, the matrix-memory recurrence, the per-head
// norm + gate, the router and the per-row expert evaluation of a routed feed-forward, and the parallel residual add.
//
// Every kernel is built for bf16 and for fp32 activations (template AT); the residual stream, norm statistics,
// attention scores and weights, router logits, gates and recurrent states are fp32 in both. Sizes are run-time values
// with no alignment assumptions. A step's rows are described by segments: seg[r] = (first row, rows, first position,
// state slot), one per sequence in the step, and tok_seg[t] = the segment of row t. A segment whose first position is
// 0 has zero state: its slot is written, never read, so reused slots need no clearing.
//
//   rms_norm        x / sqrt(mean(x^2) + eps) * w of the fp32 stream -> AT
//   kv_store        a row's key columns -> its slot of the paged keys; its value columns -> the page-wise transposed
//                   paged values [page][channel][16 tokens]
//   sigmoid_attn    one wave per (row, head): lane = key for the scores (the query row broadcast from LDS), weights
//                   sigmoid(cap(score) - distance bias + head bias), then lane = value channel, each lane reading its
//                   channel's 16 consecutive tokens of a transposed page; a row's keys are visited in order, whatever
//                   the batch
//   rglru_scan      S <- a S + sqrt(1 - a^2) i u per channel, one thread per (segment, channel), 8 rows' inputs
//                   loaded and transformed at a time
//   mlstm_scan      one workgroup per (segment, head, 63 value columns + the normaliser as a 64th): thread (dg, v) keeps
//                   a quarter of the rows of column v of the matrix memory in registers; q, k, v and gates of 8
//                   tokens are staged in LDS (double buffered), the four partial read-outs per column summed through LDS
//   head_norm_gate  unit RMS per head * weight * sigmoid(gate)
//   moe_topk        top-k of fp32 router logits by k wave-wide arg-max passes (ties: the lower index), softmax over
//                   the chosen
//   moe_gate_up / moe_down   experts evaluated per (row, chosen expert) pair: any sizes, both dtypes; the pairs of a
//                   row are summed in their order
//   add2            x += y1 + y2 (fp32), optionally with the next layer's RMS norm of the new x in the same pass
#include "common.h"

namespace kafka {
namespace hg {

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)(*p); }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + expf(-z)); }

constexpr int NT = 256;
constexpr int PAGE = 16;

// Workgroup barrier for LDS hand-overs that leaves global loads (a prefetched next block) in flight: __syncthreads()
// would drain them as well. This wave's LDS reads and writes are complete (lgkmcnt 0) before it arrives.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <typename AT>
__global__ __launch_bounds__(NT) void rms_norm_kernel(const float* __restrict__ x, int64_t xs, const AT* __restrict__ w,
                                                      float eps, AT* __restrict__ out, int64_t os, int d) {
  __shared__ float red[NT / 64];
  const float* r = x + (int64_t)blockIdx.x * xs;
  float s = 0.f;
  for (int i = threadIdx.x; i < d; i += NT) {
    const float v = r[i];
    s += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)d + eps);
  AT* o = out + (int64_t)blockIdx.x * os;
  for (int i = threadIdx.x; i < d; i += NT) stf(o + i, r[i] * rs * ldf(w + i));
}

template <typename AT>
__global__ void kv_store_kernel(const AT* __restrict__ src, int64_t ss, int k_off, int v_off, int Ck, int Cv,
                                AT* __restrict__ kc, AT* __restrict__ vt, const int64_t* __restrict__ slots, int64_t T) {
  const int C = Ck + Cv;
  const int64_t n = T * C;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / C;
    const int c = (int)(i - t * C);
    const int64_t sl = slots[t];
    if (sl < 0) continue;
    if (c < Ck) {
      kc[sl * Ck + c] = src[t * ss + k_off + c];
    } else {
      const int cv = c - Ck;
      vt[((sl / PAGE) * Cv + cv) * PAGE + (sl % PAGE)] = src[t * ss + v_off + cv];
    }
  }
}

// ---- sigmoid attention, one wave per (row, head) -----------------------------------------------------------------------
constexpr int SA_MAXD = 512;   // largest query / key head size (the query row sits in LDS as fp32)
constexpr int SA_NV = 8;       // value columns per lane: head value size <= 64 * SA_NV

struct SigParams {
  float scale, softcap, t_coef;
  double t_every;
};

// the temperature of a query at position p: 1 + coef ln(floor((p + 1) / every) + 1), the quotient in double so that
// the floor falls where it does in exact arithmetic
__device__ __forceinline__ float query_temp(int64_t p, float coef, double every) {
  if (coef == 0.f) return 1.0f;
  return 1.0f + coef * logf((float)floor((double)(p + 1) / every) + 1.0f);
}

__device__ __forceinline__ float sig_weight(float dot, float st, float cap, float r1, float r2, float pb, float dist) {
  float s = dot * st;
  if (cap > 0.f) s = cap * tanhf(s / cap);
  s -= r1 * log1pf(r2 * dist);
  return sigmoidf(s + pb);
}

template <typename AT>
__global__ __launch_bounds__(NT) void sigmoid_attn_kernel(const AT* __restrict__ q, int64_t qs, int q_off,
                                                          const AT* __restrict__ kc, const AT* __restrict__ vt,
                                                          const int* __restrict__ bt, int bt_stride,
                                                          const int* __restrict__ tok_seg,
                                                          const int64_t* __restrict__ positions, int H, int G, int D,
                                                          int Dv, SigParams sp, const float* __restrict__ r1,
                                                          const float* __restrict__ r2, const float* __restrict__ pb,
                                                          AT* __restrict__ out, int64_t os, int64_t pairs) {
  __shared__ float qsh[NT / 64][SA_MAXD];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t pair = (int64_t)blockIdx.x * (NT / 64) + wave;
  if (pair >= pairs) return;  // whole waves leave; nothing below synchronises across waves
  const int64_t t = pair / H;
  const int h = (int)(pair - t * H);
  const int g = h / (H / G);
  const int64_t p = positions[t];
  const int* pages = bt + (int64_t)tok_seg[t] * bt_stride;
  float* qw = qsh[wave];
  for (int i = lane; i < D; i += 64) qw[i] = ldf(q + t * qs + q_off + (int64_t)h * D + i);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const float st = sp.scale * query_temp(p, sp.t_coef, sp.t_every);
  const float hr1 = r1[h], hr2 = r2[h], hpb = pb[h];
  const int Ck = G * D, Cv = G * Dv;
  float acc[SA_NV];
#pragma unroll
  for (int i = 0; i < SA_NV; ++i) acc[i] = 0.f;
  for (int64_t j0 = 0; j0 <= p; j0 += 64) {
    const int64_t j = j0 + lane;
    float w = 0.f;
    if (j <= p) {
      const AT* kr = kc + ((int64_t)pages[j / PAGE] * PAGE + (j % PAGE)) * Ck + (int64_t)g * D;
      float dot = 0.f;
      for (int i = 0; i < D; ++i) dot += qw[i] * ldf(kr + i);
      w = sig_weight(dot, st, sp.softcap, hr1, hr2, hpb, (float)(p - j));
    }
    const int nk = (int)((p - j0 + 1 < 64) ? (p - j0 + 1) : 64);  // visible keys of this block
    for (int pg = 0; pg * PAGE < nk; ++pg) {
      const int64_t page = pages[(j0 >> 4) + pg];
      const int ne = (nk - pg * PAGE < PAGE) ? nk - pg * PAGE : PAGE;
      float wk[PAGE];
#pragma unroll
      for (int e = 0; e < PAGE; ++e) wk[e] = __shfl(w, pg * PAGE + e, 64);
#pragma unroll
      for (int i = 0; i < SA_NV; ++i) {
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
#pragma unroll
  for (int i = 0; i < SA_NV; ++i) {
    const int v = lane + 64 * i;
    if (v < Dv) stf(out + t * os + (int64_t)h * Dv + v, acc[i]);
  }
}

// ---- sigmoid attention on the matrix cores (bf16) ------------------------------------------------------------------
// One workgroup (4 waves) per (tile, key/value head): a tile is 32 query rows = (token, query head of this key/value
// head) pairs of consecutive tokens of one segment (floor(32 / rep) tokens, rep = H / G query heads per key/value
// head). Keys go by in blocks of 128:
//   scores   wave w takes keys 32 w .. 32 w + 31 of the block: S = Q K^T as D / 16 MFMA steps (32x32x16), the Q tile
//            read from LDS, the key rows straight from the paged cache (lane = key, 16 bytes per step), the next
//            block's rows requested before this block's weights are computed;
//   weights  per score, in fp32: cap tanh(s scale temp / cap) - r1 ln(1 + r2 distance) + head bias -> sigmoid; keys
//            ahead of the row weigh 0; P goes to LDS as bf16;
//   values   wave w owns output columns [32 TW w, 32 TW (w + 1)): O += P V with V read from the page-wise transposed
//            values (lane = column, 8 consecutive keys = 16 bytes), one page per MFMA step.
// There is no running maximum and no normaliser: the weights are what they are, and a block's product is just added.
// With gridDim.z > 1 the tile's key blocks are dealt to gridDim.z workgroups in contiguous ranges; each leaves its
// sums in po [z][T][H Dv] (fp32) and sig_reduce adds them in order. Needs 16-token pages and D % 16 == 0.
constexpr int SM_ROWS = 32;

__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

template <int TW, int NKSC>
__global__ __launch_bounds__(256) void sigmoid_attn_mfma_kernel(
    const bf16* __restrict__ q, int64_t qs, int q_off, const bf16* __restrict__ kc, const bf16* __restrict__ vt,
    const int* __restrict__ bt, int bt_stride, const int* __restrict__ items, const int64_t* __restrict__ positions,
    int H, int G, int D, int Dv, SigParams sp, const float* __restrict__ r1, const float* __restrict__ r2,
    const float* __restrict__ pb, bf16* __restrict__ out, int64_t os, float* __restrict__ po, int64_t T) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int nks = D >> 4, qstride = D + 8;
  bf16* Qs = reinterpret_cast<bf16*>(smem);                       // [32][D + 8]
  bf16* Ps = Qs + SM_ROWS * qstride;                              // [32][128 + 8]
  float* rowf = reinterpret_cast<float*>(Ps + SM_ROWS * 136);     // [4][32]: score factor, r1, r2 log2e-free, bias
  int* prow_s = reinterpret_cast<int*>(rowf + 4 * SM_ROWS);       // [32]
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, lr = lane & 31, lh = lane >> 5;
  const int t0 = items[4 * blockIdx.x], ntok = items[4 * blockIdx.x + 1], sg = items[4 * blockIdx.x + 2];
  const int g = blockIdx.y, rep = H / G;
  const int nrows = ntok * rep;
  for (int i = threadIdx.x; i < SM_ROWS * (D >> 3); i += 256) {
    const int r = i / (D >> 3), d0 = (i - r * (D >> 3)) << 3;
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (r < nrows) v = load_bf16x8(q + (int64_t)(t0 + r / rep) * qs + q_off + (int64_t)(g * rep + r % rep) * D + d0);
    store_bf16x8(Qs + r * qstride + d0, v);
  }
  if (threadIdx.x < SM_ROWS) {
    const int r = threadIdx.x;
    const bool ok = r < nrows;
    const int h = g * rep + (ok ? r % rep : 0);
    const int64_t p = ok ? positions[t0 + r / rep] : -1;   // a row beyond the tile sees no key
    prow_s[r] = (int)p;
    rowf[r] = sp.scale * query_temp(p < 0 ? 0 : p, sp.t_coef, sp.t_every);
    rowf[SM_ROWS + r] = r1[h] * 0.6931471805599453f;        // times log2 of (1 + r2 distance) below
    rowf[2 * SM_ROWS + r] = r2[h];
    rowf[3 * SM_ROWS + r] = pb[h];
  }
  const int maxpos = (int)positions[t0 + ntok - 1];
  __syncthreads();
  int prow[16];
  float fac[16];
  f32x16 O[TW];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = (i & 3) + 8 * (i >> 2) + 4 * lh;
    prow[i] = prow_s[r];
    fac[i] = rowf[r];
  }
#pragma unroll
  for (int tw = 0; tw < TW; ++tw)
#pragma unroll
    for (int i = 0; i < 16; ++i) O[tw][i] = 0.f;
  const int* btr = bt + (int64_t)sg * bt_stride;
  const int Ck = G * D, Cv = G * Dv;
  const int nblocks = (maxpos >> 7) + 1;
  const bf16* qrow = Qs + lr * qstride + 8 * lh;
  bf16x8 kf[NKSC];
  auto fetch_keys = [&](int kb) {
    const int kcix = min(kb * 128 + 32 * w + lr, maxpos);  // past the tile's last position: a valid row, masked below
    const bf16* krow = kc + ((int64_t)btr[kcix >> 4] * PAGE + (kcix & 15)) * Ck + (int64_t)g * D + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < NKSC; ++ks)
      if (ks < nks) kf[ks] = load_bf16x8(krow + 16 * ks);
  };
  const int nsplit = gridDim.z;
  const int bps = (nblocks + nsplit - 1) / nsplit;
  const int kb0 = blockIdx.z * bps, kb1 = min(nblocks, kb0 + bps);
  const float cap = sp.softcap, inv_cap2 = cap > 0.f ? 2.0f * 1.4426950408889634f / cap : 0.f;
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
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = (i & 3) + 8 * (i >> 2) + 4 * lh;
      float p = 0.f;
      if (any && key <= prow[i]) {
        float s = S[i] * fac[i];
        // cap tanh(s / cap) = cap (1 - 2 / (1 + e^(2 s / cap)))
        if (cap > 0.f) s = cap - 2.0f * cap * fast_rcp(1.0f + fast_exp2(s * inv_cap2));
        const float dist = (float)(prow[i] - key);
        s -= rowf[SM_ROWS + r] * fast_log2(1.0f + rowf[2 * SM_ROWS + r] * dist);
        s += rowf[3 * SM_ROWS + r];
        p = fast_rcp(1.0f + fast_exp2(-1.4426950408889634f * s));
      }
      Ps[r * 136 + 32 * w + lr] = (bf16)p;
    }
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
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = (i & 3) + 8 * (i >> 2) + 4 * lh;
    if (r >= nrows) continue;
    const int64_t t = t0 + r / rep;
    const int h = g * rep + r % rep;
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      const int col = (w * TW + tw) * 32 + lr;
      if (col >= Dv) continue;
      if (nsplit == 1)
        out[t * os + (int64_t)h * Dv + col] = (bf16)O[tw][i];
      else
        po[((int64_t)blockIdx.z * T + t) * ((int64_t)H * Dv) + (int64_t)h * Dv + col] = O[tw][i];
    }
  }
}

// out = sum_z po[z] over the key-range splits, in order
__global__ void sig_reduce_kernel(const float* __restrict__ po, int nsplit, int64_t T, int C, bf16* __restrict__ out,
                                  int64_t os) {
  const int64_t n = T * C;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float s = 0.f;
    for (int z = 0; z < nsplit; ++z) s += po[(int64_t)z * n + i];
    const int64_t t = i / C;
    out[t * os + (i - t * C)] = (bf16)s;
  }
}

// ---- real-gated linear recurrence ---------------------------------------------------------------------------------------
// One thread per (segment, channel) walks the segment's rows; the inputs of RG_TB rows are loaded together (independent
// loads in flight at once) and everything that does not depend on the state - both gates, the decay, the input's
// scale, the gelu branch - is computed before the short dependent chain S <- a S + b of the block.
constexpr int RG_TB = 8;

template <typename AT>
__global__ void rglru_scan_kernel(const float* __restrict__ gates, int64_t gs, const AT* __restrict__ proj, int64_t ps,
                                  const AT* __restrict__ u, int64_t us, const float* __restrict__ rate,
                                  const int* __restrict__ seg, float* __restrict__ state, AT* __restrict__ out,
                                  int64_t os, int W) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int r = blockIdx.y;
  const int q0 = seg[4 * r], n = seg[4 * r + 1], p0 = seg[4 * r + 2], slot = seg[4 * r + 3];
  float S = p0 > 0 ? state[(int64_t)slot * W + c] : 0.f;
  const float rt = rate[c];
  for (int b0 = 0; b0 < n; b0 += RG_TB) {
    const int nt = min(RG_TB, n - b0);
    float gr[RG_TB], gi[RG_TB], uu[RG_TB], yy[RG_TB];
#pragma unroll
    for (int j = 0; j < RG_TB; ++j) {
      const int64_t t = (int64_t)q0 + b0 + (j < nt ? j : 0);
      gr[j] = gates[t * gs + c];
      gi[j] = gates[t * gs + W + c];
      uu[j] = ldf(u + t * us + c);
      yy[j] = ldf(proj + t * ps + c);
    }
    float a[RG_TB], in[RG_TB];
#pragma unroll
    for (int j = 0; j < RG_TB; ++j) {
      const float la = rt * sigmoidf(gr[j]);
      a[j] = expf(la);
      in[j] = sqrtf(-expm1f(2.0f * la)) * sigmoidf(gi[j]) * uu[j];
      yy[j] = gelu_tanh(yy[j]);
    }
#pragma unroll
    for (int j = 0; j < RG_TB; ++j) {
      if (j < nt) {
        S = a[j] * S + in[j];
        stf(out + ((int64_t)q0 + b0 + j) * os + c, S * yy[j]);
      }
    }
  }
  state[(int64_t)slot * W + c] = S;
}

// The recurrence for long segments, in four launches that leave only multiply-adds in the sequential part:
//   prep     per (row, channel), all in parallel: a = exp(rate sigmoid(g_r)) and b = sqrt(1 - a^2) sigmoid(g_i) u replace
//            the two gate pre-activations in place;
//   local    per (segment, chunk of RG_CH rows, channel): A = prod a and the chunk's scan from zero, B;
//   carry    per (segment, channel), over the segment's chunks in order: entry state E_c, S <- A_c S + B_c; the last S is
//            the sequence's new state;
//   apply    per (segment, chunk, channel): the scan again from E_c, out = S * gelu(branch), rounded once as in the
//            row-by-row kernel.
// The result differs from the row-by-row order only by fp32 rounding (the chunks' entry states are re-associated).
constexpr int RG_CH = 64;

template <typename AT>
__global__ void rglru_prep_kernel(float* __restrict__ gates, int64_t gs, const AT* __restrict__ u, int64_t us,
                                  const float* __restrict__ rate, int64_t T, int W) {
  const int64_t n = T * W;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / W;
    const int c = (int)(i - t * W);
    const float la = rate[c] * sigmoidf(gates[t * gs + c]);
    const float b = sqrtf(-expm1f(2.0f * la)) * sigmoidf(gates[t * gs + W + c]) * ldf(u + t * us + c);
    gates[t * gs + c] = expf(la);
    gates[t * gs + W + c] = b;
  }
}

// MODE 0: local (A, B of the chunk from zero -> ab[((r * nch + ch) * 2 + {0, 1}) * W + c]); MODE 1: apply (from the
// entry state in ab[...][0], out = S * gelu(branch))
template <typename AT, int MODE>
__global__ void rglru_chunk_kernel(const float* __restrict__ gates, int64_t gs, const AT* __restrict__ proj, int64_t ps,
                                   const int* __restrict__ seg, int nch, float* __restrict__ ab, AT* __restrict__ out,
                                   int64_t os, int W) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ch = blockIdx.y, r = blockIdx.z;
  const int q0 = seg[4 * r], n = seg[4 * r + 1];
  if (c >= W || ch * RG_CH >= n) return;
  const int nt = min(RG_CH, n - ch * RG_CH);
  float* slot = ab + ((int64_t)(r * nch + ch) * 2) * W + c;
  float S = MODE == 1 ? slot[0] : 0.f, A = 1.f;
  for (int b0 = 0; b0 < nt; b0 += RG_TB) {
    float a[RG_TB], b[RG_TB], y[RG_TB];
#pragma unroll
    for (int j = 0; j < RG_TB; ++j) {
      const int64_t t = (int64_t)q0 + ch * RG_CH + b0 + (b0 + j < nt ? j : 0);
      a[j] = gates[t * gs + c];
      b[j] = gates[t * gs + W + c];
      if (MODE == 1) y[j] = ldf(proj + t * ps + c);
    }
    if (MODE == 1) {
#pragma unroll
      for (int j = 0; j < RG_TB; ++j) y[j] = gelu_tanh(y[j]);
    }
#pragma unroll
    for (int j = 0; j < RG_TB; ++j) {
      if (b0 + j < nt) {
        S = a[j] * S + b[j];
        if (MODE == 0) A *= a[j];
        if (MODE == 1) stf(out + ((int64_t)q0 + ch * RG_CH + b0 + j) * os + c, S * y[j]);
      }
    }
  }
  if (MODE == 0) {
    slot[0] = A;
    slot[W] = S;
  }
}

__global__ void rglru_carry_kernel(const int* __restrict__ seg, int nch, float* __restrict__ ab,
                                   float* __restrict__ state, int W) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int r = blockIdx.y;
  const int n = seg[4 * r + 1], p0 = seg[4 * r + 2], slot = seg[4 * r + 3];
  float S = p0 > 0 ? state[(int64_t)slot * W + c] : 0.f;
  const int used = (n + RG_CH - 1) / RG_CH;
  for (int ch = 0; ch < used; ++ch) {
    float* s2 = ab + ((int64_t)(r * nch + ch) * 2) * W + c;
    const float A = s2[0], B = s2[W];
    s2[0] = S;   // the chunk's entry state
    S = A * S + B;
  }
  state[(int64_t)slot * W + c] = S;
}

// ---- matrix memory --------------------------------------------------------------------------------------------------------
constexpr int ML_VS = 63;  // value columns of a workgroup; its 64th lane carries the normaliser as one more column
constexpr int ML_DG = 4;   // row groups (one wave each)
constexpr int ML_TB = 8;   // tokens per staged block

// One workgroup per (segment, head, 63 value columns). Thread (dg, vv) keeps rows d = dg RD .. dg RD + RD - 1 of column vv
// of the matrix memory in registers; lane 63 of every wave keeps the same rows of the normaliser n, which is the memory's
// update with a value of 1 - so n . q falls out as that column's read-out. The inputs of ML_TB tokens are staged in
// LDS at a time (q scaled, k, the value slice, the transformed gates), double buffered, the next block's global loads
// in flight while this block is scanned: the threads walk the block's tokens without synchronising (the memory is
// thread-private), leave ML_DG partial read-outs per (token, column) in LDS, and after one barrier the partials are
// summed and divided. Two barriers per block.
template <typename AT, int RD>
__global__ __launch_bounds__(NT) void mlstm_scan_kernel(const AT* __restrict__ qkv, int64_t qs,
                                                        const float* __restrict__ gates, int64_t gs, int H, int D,
                                                        int Dv, float cap, const int* __restrict__ seg,
                                                        float* __restrict__ Sst, float* __restrict__ nst,
                                                        float* __restrict__ mst, float* __restrict__ out, int64_t os) {
  constexpr int DMAX = ML_DG * RD;
  constexpr int NQK = (2 * DMAX * ML_TB + NT - 1) / NT;   // staged q | k elements per thread
  constexpr int NV = (64 * ML_TB + NT - 1) / NT;          // staged value elements per thread
  __shared__ __attribute__((aligned(16))) float qk[2][ML_TB][2][DMAX];
  __shared__ float vs[2][ML_TB][64];
  __shared__ float gsh[2][ML_TB][2];
  __shared__ float part[ML_TB][ML_DG][64];
  __shared__ float msh[ML_TB];
  const int r = blockIdx.z, h = blockIdx.y, v0 = blockIdx.x * ML_VS;
  const int q0 = seg[4 * r], n = seg[4 * r + 1], p0 = seg[4 * r + 2], slot = seg[4 * r + 3];
  const int dg = threadIdx.x >> 6, vv = threadIdx.x & 63;
  const bool is_n = vv == ML_VS;                 // the normaliser's lane
  const bool vok = !is_n && v0 + vv < Dv;
  float S[RD];
  float* Sp = Sst + (((int64_t)slot * H + h) * D) * Dv + v0 + vv;
  float* np = nst + ((int64_t)slot * H + h) * D;
  float m = 0.f;
#pragma unroll
  for (int i = 0; i < RD; ++i) {
    const int d = dg * RD + i;
    S[i] = 0.f;
    if (p0 > 0 && d < D) {
      if (vok) S[i] = Sp[(int64_t)d * Dv];
      if (is_n) S[i] = np[d];
    }
  }
  if (p0 > 0) m = mst[(int64_t)slot * H + h];
  const float qscale = 1.0f / sqrtf((float)D);
  const int qo = h * D, ko = H * D + h * D, vo = 2 * H * D + h * Dv + v0;
  const int nblk = (n + ML_TB - 1) / ML_TB;
  float pqk[NQK], pv[NV], pg = 0.f;
  auto fetch = [&](int blk) {   // global loads of a block into registers
    const int64_t t0 = (int64_t)q0 + blk * ML_TB;
    const int nt = min(ML_TB, n - blk * ML_TB);
#pragma unroll
    for (int e = 0; e < NQK; ++e) {
      const int idx = threadIdx.x + NT * e;
      const int j = idx / (2 * DMAX), rr = idx - j * 2 * DMAX, which = rr / DMAX, d = rr - which * DMAX;
      pqk[e] = (j < nt && d < D) ? ldf(qkv + (t0 + j) * qs + (which ? ko : qo) + d) : 0.f;
    }
#pragma unroll
    for (int e = 0; e < NV; ++e) {
      const int idx = threadIdx.x + NT * e;
      const int j = idx >> 6, c = idx & 63;
      pv[e] = (j < nt && c < ML_VS && v0 + c < Dv) ? ldf(qkv + (t0 + j) * qs + vo + c) : (c == ML_VS ? 1.0f : 0.f);
    }
    if (threadIdx.x < 2 * ML_TB) {
      const int j = threadIdx.x >> 1, w = threadIdx.x & 1;
      pg = j < nt ? gates[(t0 + j) * gs + w * H + h] : 0.f;
    }
  };
  auto stage = [&](int buf) {   // registers -> LDS (q scaled, gates transformed)
#pragma unroll
    for (int e = 0; e < NQK; ++e) {
      const int idx = threadIdx.x + NT * e;
      const int j = idx / (2 * DMAX), rr = idx - j * 2 * DMAX, which = rr / DMAX, d = rr - which * DMAX;
      if (j < ML_TB) qk[buf][j][which][d] = which ? pqk[e] : pqk[e] * qscale;
    }
#pragma unroll
    for (int e = 0; e < NV; ++e) {
      const int idx = threadIdx.x + NT * e;
      if ((idx >> 6) < ML_TB) vs[buf][idx >> 6][idx & 63] = pv[e];
    }
    if (threadIdx.x < 2 * ML_TB) {
      const int j = threadIdx.x >> 1, w = threadIdx.x & 1;
      const float z = cap * tanhf(pg / cap);
      gsh[buf][j][w] = w ? fminf(z, 0.f) - log1pf(expf(-fabsf(z))) : z;   // forget: logsigmoid, input: as is
    }
  };
  fetch(0);
  stage(0);
  for (int blk = 0; blk < nblk; ++blk) {
    const int buf = blk & 1;
    const int nt = min(ML_TB, n - blk * ML_TB);
    if (blk + 1 < nblk) fetch(blk + 1);
    lds_barrier();     // this block's staged inputs are visible; the other buffer and `part` are free
#pragma unroll 1
    for (int j = 0; j < nt; ++j) {   // (one token at a time: unrolling this loop too would not fit the registers)
      const float ig = gsh[buf][j][0], fg = gsh[buf][j][1];
      const float mn = fmaxf(fg + m, ig);
      const float dec = expf(fg + m - mn), gain = expf(ig - mn);
      m = mn;
      const float gv = gain * vs[buf][j][vv];
      const f32x4* qv = reinterpret_cast<const f32x4*>(&qk[buf][j][0][dg * RD]);
      const f32x4* kv = reinterpret_cast<const f32x4*>(&qk[buf][j][1][dg * RD]);
      float po = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < RD / 4; ++i4) {   // rows past D hold zeros in q and k: their memory stays zero
        const f32x4 q4 = qv[i4], k4 = kv[i4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[4 * i4 + e] = dec * S[4 * i4 + e] + gv * k4[e];
          po += S[4 * i4 + e] * q4[e];
        }
      }
      part[j][dg][vv] = po;
      if (threadIdx.x == 0) msh[j] = m;
    }
    if (blk + 1 < nblk) stage(buf ^ 1);
    lds_barrier();     // the partial read-outs are complete
    for (int idx = threadIdx.x; idx < nt * 64; idx += NT) {
      const int j = idx >> 6, c = idx & 63;
      if (c < ML_VS && v0 + c < Dv) {
        float o = 0.f, nq = 0.f;
#pragma unroll
        for (int k = 0; k < ML_DG; ++k) {
          o += part[j][k][c];
          nq += part[j][k][ML_VS];
        }
        const int64_t t = (int64_t)q0 + blk * ML_TB + j;
        out[t * os + (int64_t)h * Dv + v0 + c] = o / (fmaxf(fabsf(nq), expf(-msh[j])) + 1e-6f);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < RD; ++i) {
    const int d = dg * RD + i;
    if (d < D) {
      if (vok) Sp[(int64_t)d * Dv] = S[i];
      if (is_n && blockIdx.x == 0) np[d] = S[i];
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) mst[(int64_t)slot * H + h] = m;
}

template <typename AT>
__global__ __launch_bounds__(NT) void head_norm_gate_kernel(const float* __restrict__ o, int64_t os_,
                                                            const AT* __restrict__ w, const AT* __restrict__ g,
                                                            int64_t gs, int g_off, int H, int Dv, float eps,
                                                            AT* __restrict__ out, int64_t outs, int64_t pairs,
                                                            float scale) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t pair = (int64_t)blockIdx.x * (NT / 64) + wave;
  if (pair >= pairs) return;
  const int64_t t = pair / H;
  const int h = (int)(pair - t * H);
  const float* r = o + t * os_ + (int64_t)h * Dv;
  float s = 0.f;
  for (int i = lane; i < Dv; i += 64) s += r[i] * r[i];
  const float rs = 1.0f / sqrtf(wave_sum(s) / (float)Dv + eps);
  for (int i = lane; i < Dv; i += 64) {
    const int c = h * Dv + i;
    float v = r[i] * rs * ldf(w + c) * scale;
    if (g != nullptr) v *= sigmoidf(ldf(g + t * gs + g_off + c));
    stf(out + t * outs + c, v);
  }
}

// ---- routed feed-forward ---------------------------------------------------------------------------------------------------
constexpr int RT_MAXE = 512;  // experts (8 per lane)
constexpr int RT_MAXK = 16;

// top-k of fp32 router logits [T, E] (one wave per row: k wave-wide arg-max passes, ties to the lower index) and the
// softmax over the chosen logits
__global__ __launch_bounds__(NT) void moe_topk_kernel(const float* __restrict__ logits, int64_t ls, int E, int k,
                                                      float* __restrict__ tw, int* __restrict__ te, int64_t T) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * (NT / 64) + wave;
  if (t >= T) return;
  float z[RT_MAXE / 64];
#pragma unroll
  for (int i = 0; i < RT_MAXE / 64; ++i) {
    const int e = lane + 64 * i;
    z[i] = e < E ? logits[t * ls + e] : -INFINITY;
  }
  float val[RT_MAXK];
  for (int j = 0; j < k; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < RT_MAXE / 64; ++i) {
      const int e = lane + 64 * i;
      if (e < E && (z[i] > bv || (z[i] == bv && e < bi))) { bv = z[i]; bi = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
#pragma unroll
    for (int i = 0; i < RT_MAXE / 64; ++i)
      if (bi == lane + 64 * i) z[i] = -INFINITY;
    if (j < RT_MAXK) val[j] = bv;
    if (lane == 0) te[t * k + j] = bi;
  }
  if (lane == 0) {
    float sum = 0.f;
    for (int j = 0; j < k; ++j) sum += expf(val[j] - val[0]);
    for (int j = 0; j < k; ++j) tw[t * k + j] = expf(val[j] - val[0]) / sum;
  }
}

constexpr int MOE_MAXD = 8192;  // the row sits in LDS as fp32

// a[pair][f] = act(W_gate[e] h, W_up[e] h): one workgroup per (pair, block of FB rows), one wave per row.
// act(g, u) = silu(g) u, or with limit > 0 the clamped form g' sigmoid(alpha g') (u' + 1), g' = min(g, limit),
// u' = clamp(u, -limit, limit).
__device__ __forceinline__ float glu_act(float g, float u, float limit, float alpha) {
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
  }
  return g / (1.0f + expf(-g)) * u;
}

template <typename AT>
__global__ __launch_bounds__(NT) void moe_gate_up_kernel(const AT* __restrict__ h, int64_t hs,
                                                         const AT* __restrict__ wgu, const int* __restrict__ te, int d,
                                                         int F, int k, int FB, AT* __restrict__ a, float limit,
                                                         float alpha) {
  extern __shared__ float hsh[];
  const int64_t pair = blockIdx.x;
  const int64_t t = pair / k;
  const int e = te[pair];
  for (int i = threadIdx.x; i < d; i += NT) hsh[i] = ldf(h + t * hs + i);
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const AT* wg = wgu + (int64_t)e * 2 * F * d;
  const int f1 = min(F, (int)(blockIdx.y + 1) * FB);
  for (int f = blockIdx.y * FB + wave; f < f1; f += NT / 64) {
    const AT* g = wg + (int64_t)f * d;
    const AT* u = wg + (int64_t)(F + f) * d;
    float sg = 0.f, su = 0.f;
    for (int i = lane; i < d; i += 64) {
      const float x = hsh[i];
      sg += x * ldf(g + i);
      su += x * ldf(u + i);
    }
    sg = wave_sum(sg);
    su = wave_sum(su);
    if (lane == 0) stf(a + pair * F + f, glu_act(sg, su, limit, alpha));
  }
}

// out[t][c] = sum_j tw[t][j] W_down[e_j][c] . a[t k + j]: one workgroup per (row, block of CB columns); the row's
// activations are staged one chosen expert at a time
constexpr int MOE_CPW = 16;   // output columns a wave accumulates in registers across the experts

template <typename AT>
__global__ __launch_bounds__(NT) void moe_down_kernel(const AT* __restrict__ a, const AT* __restrict__ wd,
                                                      const float* __restrict__ tw, const int* __restrict__ te, int d,
                                                      int F, int k, int CB, float* __restrict__ out, int64_t os) {
  extern __shared__ float ash[];  // [F]
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c0 = blockIdx.y * CB, c1 = min(d, c0 + CB);   // CB <= MOE_CPW * (NT / 64): every column has a register
  float acc[MOE_CPW];
#pragma unroll
  for (int i = 0; i < MOE_CPW; ++i) acc[i] = 0.f;
  for (int j = 0; j < k; ++j) {
    __syncthreads();
    for (int i = threadIdx.x; i < F; i += NT) ash[i] = ldf(a + (t * k + j) * F + i);
    __syncthreads();
    const AT* we = wd + (int64_t)te[t * k + j] * d * F;
    const float wj = tw[t * k + j];
#pragma unroll
    for (int i = 0; i < MOE_CPW; ++i) {
      const int c = c0 + wave + (NT / 64) * i;
      if (c < c1) {
        const AT* wr = we + (int64_t)c * F;
        float s = 0.f;
        for (int f = lane; f < F; f += 64) s += ash[f] * ldf(wr + f);
        acc[i] += wj * wave_sum(s);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MOE_CPW; ++i) {
    const int c = c0 + wave + (NT / 64) * i;
    if (c < c1 && lane == 0) out[t * os + c] = acc[i];
  }
}

template <typename AT, typename BT>
__global__ void add2_kernel(float* __restrict__ x, int64_t xs, const AT* __restrict__ y1, int64_t s1,
                            const BT* __restrict__ y2, int64_t s2, int64_t T, int d) {
  const int64_t n = T * d;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / d;
    const int c = (int)(i - t * d);
    float s = ldf(y1 + t * s1 + c);
    if (y2) s += ldf(y2 + t * s2 + c);
    x[t * xs + c] += s;
  }
}

// x += y1 + y2 and, in the same pass over the row, out = rms_norm(x) * w (the next layer's norm): one workgroup per row
template <typename AT, typename BT>
__global__ __launch_bounds__(NT) void add2_norm_kernel(float* __restrict__ x, int64_t xs, const AT* __restrict__ y1,
                                                       int64_t s1, const BT* __restrict__ y2, int64_t s2,
                                                       const AT* __restrict__ w, float eps, AT* __restrict__ out,
                                                       int64_t os, int d) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  float* r = x + t * xs;
  float acc = 0.f;
  for (int i = threadIdx.x; i < d; i += NT) {
    float s = ldf(y1 + t * s1 + i);
    if (y2) s += ldf(y2 + t * s2 + i);
    const float v = r[i] + s;
    r[i] = v;
    acc += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum<NT>(acc, red) / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += NT) stf(out + t * os + i, r[i] * rs * ldf(w + i));  // (this thread's own writes)
}

static inline int ew_grid(int64_t n) { return (int)std::min<int64_t>((n + 255) / 256, 65535 * 4); }

}  // namespace hg
}  // namespace kafka

using namespace kafka::hg;

#define DISPATCH_AT(f32, ...)             \
  if (f32) {                              \
    using AT = float;                     \
    __VA_ARGS__;                          \
  } else {                                \
    using AT = bf16;                      \
    __VA_ARGS__;                          \
  }

extern "C" {

hipError_t kafka_hy_rms_norm(int f32, const float* x, int64_t xs, const void* w, float eps, void* out, int64_t os,
                             int T, int d, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  DISPATCH_AT(f32, { rms_norm_kernel<AT><<<T, NT, 0, st>>>(x, xs, (const AT*)w, eps, (AT*)out, os, d); });
  return hipGetLastError();
}

hipError_t kafka_hy_kv_store(int f32, const void* src, int64_t ss, int k_off, int v_off, int Ck, int Cv, void* kc,
                             void* vt, const int64_t* slots, int64_t T, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  DISPATCH_AT(f32, {
    kv_store_kernel<AT><<<ew_grid(T * (Ck + Cv)), 256, 0, st>>>((const AT*)src, ss, k_off, v_off, Ck, Cv, (AT*)kc,
                                                               (AT*)vt, slots, T);
  });
  return hipGetLastError();
}

int kafka_hy_sigmoid_attn_max_d() { return SA_MAXD; }
int kafka_hy_sigmoid_attn_max_dv() { return 64 * SA_NV; }

hipError_t kafka_hy_sigmoid_attn(int f32, const void* q, int64_t qs, int q_off, const void* kc, const void* vt,
                                 const int* bt, int bt_stride, const int* tok_seg, const int64_t* positions, int H,
                                 int G, int D, int Dv, float scale, float softcap, float t_coef, double t_every,
                                 const float* r1, const float* r2, const float* pb, void* out, int64_t os, int64_t T,
                                 hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (D > SA_MAXD || Dv > 64 * SA_NV || G < 1 || H % G) return hipErrorInvalidValue;
  const SigParams sp{scale, softcap, t_coef, t_every};
  const int64_t pairs = T * H;
  const int grid = (int)((pairs + NT / 64 - 1) / (NT / 64));
  DISPATCH_AT(f32, {
    sigmoid_attn_kernel<AT><<<grid, NT, 0, st>>>((const AT*)q, qs, q_off, (const AT*)kc, (const AT*)vt, bt, bt_stride,
                                                 tok_seg, positions, H, G, D, Dv, sp, r1, r2, pb, (AT*)out, os, pairs);
  });
  return hipGetLastError();
}

// bf16 shapes the matrix-core kernel takes (else the per-wave kernel above runs)
int kafka_hy_sigmoid_attn_mfma_ok(int page, int D, int Dv, int rep) {
  return page == PAGE && D >= 16 && D % 16 == 0 && D <= 256 && Dv >= 1 && Dv <= 256 && rep >= 1 && rep <= SM_ROWS;
}

hipError_t kafka_hy_sigmoid_attn_mfma(const void* q, int64_t qs, int q_off, const void* kc, const void* vt,
                                      const int* bt, int bt_stride, const int* items, int n_items,
                                      const int64_t* positions, int H, int G, int D, int Dv, float scale,
                                      float softcap, float t_coef, double t_every, const float* r1, const float* r2,
                                      const float* pb, void* out, int64_t os, int nsplit, float* po, int64_t T,
                                      hipStream_t st) {
  if (n_items <= 0) return hipSuccess;
  if (G < 1 || H % G || !kafka_hy_sigmoid_attn_mfma_ok(PAGE, D, Dv, H / G)) return hipErrorInvalidValue;
  if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && po == nullptr)) return hipErrorInvalidValue;
  const SigParams sp{scale, softcap, t_coef, t_every};
  const size_t lds = (size_t)SM_ROWS * (D + 8) * 2 + SM_ROWS * 136 * 2 + 5 * SM_ROWS * 4;
  const dim3 grid((unsigned)n_items, (unsigned)G, (unsigned)nsplit);
  auto a = [&](auto k) {
    k<<<grid, 256, lds, st>>>((const bf16*)q, qs, q_off, (const bf16*)kc, (const bf16*)vt, bt, bt_stride, items,
                              positions, H, G, D, Dv, sp, r1, r2, pb, (bf16*)out, os, po, T);
  };
  const int nks = D / 16, tw = ((Dv + 31) / 32 + 3) / 4;
  if (tw == 1 && nks <= 4) a(sigmoid_attn_mfma_kernel<1, 4>);
  else if (tw == 1 && nks <= 8) a(sigmoid_attn_mfma_kernel<1, 8>);
  else if (tw == 1) a(sigmoid_attn_mfma_kernel<1, 16>);
  else if (nks <= 8) a(sigmoid_attn_mfma_kernel<2, 8>);
  else a(sigmoid_attn_mfma_kernel<2, 16>);
  if (nsplit > 1)
    sig_reduce_kernel<<<ew_grid(T * H * Dv), 256, 0, st>>>(po, nsplit, T, H * Dv, (bf16*)out, os);
  return hipGetLastError();
}

hipError_t kafka_hy_rglru_scan(int f32, const float* gates, int64_t gs, const void* proj, int64_t ps, const void* u,
                               int64_t us, const float* rate, const int* seg, int R, float* state, void* out,
                               int64_t os, int W, hipStream_t st) {
  if (R <= 0 || W <= 0) return hipSuccess;
  const dim3 grid((W + 63) / 64, R);
  DISPATCH_AT(f32, {
    rglru_scan_kernel<AT><<<grid, 64, 0, st>>>(gates, gs, (const AT*)proj, ps, (const AT*)u, us, rate, seg, state,
                                                (AT*)out, os, W);
  });
  return hipGetLastError();
}

int kafka_hy_rglru_chunk() { return RG_CH; }

// the chunked form: `ab` is scratch of R * nch * 2 * W floats, nch >= the longest segment's chunks of RG_CH rows
hipError_t kafka_hy_rglru_scan_chunked(int f32, float* gates, int64_t gs, const void* proj, int64_t ps, const void* u,
                                       int64_t us, const float* rate, const int* seg, int R, int nch, float* ab,
                                       float* state, void* out, int64_t os, int64_t T, int W, hipStream_t st) {
  if (R <= 0 || W <= 0 || T <= 0) return hipSuccess;
  if (nch < 1 || ab == nullptr || nch > 65535 || R > 65535) return hipErrorInvalidValue;
  const dim3 gc((W + 63) / 64, nch, R), gk((W + 63) / 64, R);
  DISPATCH_AT(f32, {
    rglru_prep_kernel<AT><<<ew_grid(T * W), 256, 0, st>>>(gates, gs, (const AT*)u, us, rate, T, W);
    rglru_chunk_kernel<AT, 0><<<gc, 64, 0, st>>>(gates, gs, (const AT*)proj, ps, seg, nch, ab, (AT*)out, os, W);
    rglru_carry_kernel<<<gk, 64, 0, st>>>(seg, nch, ab, state, W);
    rglru_chunk_kernel<AT, 1><<<gc, 64, 0, st>>>(gates, gs, (const AT*)proj, ps, seg, nch, ab, (AT*)out, os, W);
  });
  return hipGetLastError();
}

int kafka_hy_mlstm_max_d() { return ML_DG * 64; }

hipError_t kafka_hy_mlstm_scan(int f32, const void* qkv, int64_t qs, const float* gates, int64_t gs, int H, int D,
                               int Dv, float cap, const int* seg, int R, float* S, float* nrm, float* mx, float* out,
                               int64_t os, hipStream_t st) {
  if (R <= 0) return hipSuccess;
  if (D > ML_DG * 64 || D < 1 || Dv < 1) return hipErrorInvalidValue;
  const dim3 grid((Dv + ML_VS - 1) / ML_VS, H, R);
#define ML_LAUNCH(RD)                                                                                              \
  mlstm_scan_kernel<AT, RD><<<grid, NT, 0, st>>>((const AT*)qkv, qs, gates, gs, H, D, Dv, cap, seg, S, nrm, mx, out, os)
  DISPATCH_AT(f32, {
    if (D <= ML_DG * 16) ML_LAUNCH(16);
    else if (D <= ML_DG * 32) ML_LAUNCH(32);
    else ML_LAUNCH(64);
  });
#undef ML_LAUNCH
  return hipGetLastError();
}

hipError_t kafka_hy_head_norm_gate(int f32, const float* o, int64_t os_, const void* w, const void* g, int64_t gs,
                                   int g_off, int H, int Dv, float eps, void* out, int64_t outs, int64_t T,
                                   float scale, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  const int64_t pairs = T * H;
  const int grid = (int)((pairs + NT / 64 - 1) / (NT / 64));
  DISPATCH_AT(f32, {
    head_norm_gate_kernel<AT><<<grid, NT, 0, st>>>(o, os_, (const AT*)w, (const AT*)g, gs, g_off, H, Dv, eps, (AT*)out,
                                                   outs, pairs, scale);
  });
  return hipGetLastError();
}

int kafka_hy_router_max_e() { return RT_MAXE; }
int kafka_hy_router_max_k() { return RT_MAXK; }

hipError_t kafka_hy_moe_topk(const float* logits, int64_t ls, int E, int k, float* tw, int* te, int64_t T,
                             hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (E > RT_MAXE || k > RT_MAXK || k < 1 || k > E) return hipErrorInvalidValue;
  const int grid = (int)((T + NT / 64 - 1) / (NT / 64));
  moe_topk_kernel<<<grid, NT, 0, st>>>(logits, ls, E, k, tw, te, T);
  return hipGetLastError();
}

int kafka_hy_moe_rows_max_d() { return MOE_MAXD; }

hipError_t kafka_hy_moe_rows(int f32, const void* h, int64_t hs, const void* wgu, const void* wd, const float* tw,
                             const int* te, int d, int F, int k, void* a, float* out, int64_t os, int64_t T,
                             float limit, float alpha, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (d > MOE_MAXD || F > MOE_MAXD) return hipErrorInvalidValue;
  // enough workgroups for a step of few rows, many rows per workgroup for a step of many; the down kernel keeps a
  // column block's sums in registers: at most MOE_CPW columns per wave
  const int64_t pairs = T * k;
  int fb = F, cb = std::min(d, MOE_CPW * (NT / 64));
  while (pairs * ((F + fb - 1) / fb) < 1024 && fb > 8) fb = (fb + 1) / 2;
  while (T * ((d + cb - 1) / cb) < 1024 && cb > 8) cb = (cb + 1) / 2;
  const dim3 g1((unsigned)pairs, (F + fb - 1) / fb), g2((unsigned)T, (d + cb - 1) / cb);
  DISPATCH_AT(f32, {
    moe_gate_up_kernel<AT><<<g1, NT, d * sizeof(float), st>>>((const AT*)h, hs, (const AT*)wgu, te, d, F, k, fb, (AT*)a,
                                                              limit, alpha);
    moe_down_kernel<AT><<<g2, NT, (size_t)F * sizeof(float), st>>>((const AT*)a, (const AT*)wd, tw, te, d, F, k, cb,
                                                                       out, os);
  });
  return hipGetLastError();
}

hipError_t kafka_hy_add2(int f32, float* x, int64_t xs, const void* y1, int64_t s1, const void* y2, int64_t s2,
                         int y2_f32, int64_t T, int d, const void* w, float eps, void* out, int64_t os, hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (w != nullptr) {
    DISPATCH_AT(f32, {
      if (y2_f32 || !y2)
        add2_norm_kernel<AT, float><<<(unsigned)T, NT, 0, st>>>(x, xs, (const AT*)y1, s1, (const float*)y2, s2,
                                                                (const AT*)w, eps, (AT*)out, os, d);
      else
        add2_norm_kernel<AT, AT><<<(unsigned)T, NT, 0, st>>>(x, xs, (const AT*)y1, s1, (const AT*)y2, s2, (const AT*)w,
                                                             eps, (AT*)out, os, d);
    });
    return hipGetLastError();
  }
  DISPATCH_AT(f32, {
    if (y2_f32 || !y2)
      add2_kernel<AT, float><<<ew_grid(T * d), 256, 0, st>>>(x, xs, (const AT*)y1, s1, (const float*)y2, s2, T, d);
    else
      add2_kernel<AT, AT><<<ew_grid(T * d), 256, 0, st>>>(x, xs, (const AT*)y1, s1, (const AT*)y2, s2, T, d);
  });
  return hipGetLastError();
}

}  // extern "C"
