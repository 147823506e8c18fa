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
//                       per row; a row's read values stay in registers between the statistics and the scaling.
//   swish_clamp_mul     g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit)
//   qk_norm_rope_store  RMS norm over the whole q and the whole k projection, rotation of dimension pairs (2i, 2i + 1),
//                       value mix with an earlier layer's values, paged key / transposed value store
//   window_attn         softmax attention with a sliding window and a sink logit; one wave per (row, head): lane = key
//                       for the scores (the query row broadcast from LDS), online softmax over 64-key blocks, then
//                       lane = value channel reading its channel's 16 consecutive tokens of a transposed page; a
//                       row's keys are visited in order, whatever the batch
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

// ---- residual streams ----------------------------------------------------------------------------------------------
constexpr int SMAX = 8;    // streams
constexpr int UREG = 16;   // read values a thread keeps between the two passes (rows up to NT * UREG wide; wider rows
                           // recompute them from the streams just written)

template <int S>
__global__ __launch_bounds__(NT) void stream_step_kernel(float* __restrict__ xs, int64_t s_stride, int64_t t_stride,
                                                         const void* __restrict__ y, int64_t ys, bool y_f32,
                                                         const void* __restrict__ y2, int64_t y2s, bool y2_f32,
                                                         const float* __restrict__ row_scale,
                                                         const float* __restrict__ mix, const float* __restrict__ wr,
                                                         const float* __restrict__ rd, const float* __restrict__ nw,
                                                         float eps, void* __restrict__ out, int64_t os, bool out_f32,
                                                         float* __restrict__ total, int64_t ts, int d) {
  __shared__ float red[NT / 64];
  __shared__ float cM[SMAX * SMAX], cb[SMAX], ca[SMAX];
  const int64_t t = blockIdx.x;
  if (threadIdx.x < S * S && mix != nullptr) cM[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    if (wr != nullptr) cb[threadIdx.x] = wr[threadIdx.x];
    if (rd != nullptr) ca[threadIdx.x] = rd[threadIdx.x];
  }
  __syncthreads();
  float* xr = xs + t * t_stride;
  const float rs2 = y2 != nullptr ? row_scale[t] : 0.f;
  float ureg[UREG];
  float acc = 0.f;
  int it = 0;
  for (int i = threadIdx.x; i < d; i += NT, ++it) {
    float x[S];
#pragma unroll
    for (int s = 0; s < S; ++s) x[s] = xr[s * s_stride + i];
    if (mix != nullptr) {
      float yv = ldx(y, y_f32, t * ys + i);
      if (y2 != nullptr) yv += rs2 * ldx(y2, y2_f32, t * y2s + i);
      float nx[S];
#pragma unroll
      for (int r = 0; r < S; ++r) {
        float v = cb[r] * yv;
#pragma unroll
        for (int s = 0; s < S; ++s) v += cM[s * S + r] * x[s];
        nx[r] = v;
      }
#pragma unroll
      for (int s = 0; s < S; ++s) {
        x[s] = nx[s];
        xr[s * s_stride + i] = nx[s];
      }
    }
    if (total != nullptr) {
      float v = 0.f;
#pragma unroll
      for (int s = 0; s < S; ++s) v += x[s];
      total[t * ts + i] = v;
    }
    if (rd != nullptr) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < S; ++s) u += ca[s] * x[s];
      acc += u * u;
      if (it < UREG) ureg[it] = u;
    }
  }
  if (rd == nullptr) return;
  const float rs = 1.0f / sqrtf(block_sum<NT>(acc, red) / (float)d + eps);
  it = 0;
  for (int i = threadIdx.x; i < d; i += NT, ++it) {
    float u;
    if (it < UREG) {
      u = ureg[it];
    } else {  // (this thread's own writes of the first pass)
      u = 0.f;
#pragma unroll
      for (int s = 0; s < S; ++s) u += ca[s] * xr[s * s_stride + i];
    }
    const float v = u * rs * nw[i];
    if (out_f32) reinterpret_cast<float*>(out)[t * os + i] = v;
    else reinterpret_cast<bf16*>(out)[t * os + i] = (bf16)v;
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
constexpr int WA_MAXD = 512;  // query / key size (the query row sits in LDS as fp32)
constexpr int WA_NV = 8;      // value size up to 64 * WA_NV

template <typename AT>
__global__ __launch_bounds__(NT) void window_attn_kernel(const AT* __restrict__ q, int64_t qs,
                                                         const AT* __restrict__ kc, const AT* __restrict__ vt,
                                                         const int* __restrict__ bt, int bt_stride,
                                                         const int* __restrict__ tok_seg,
                                                         const int64_t* __restrict__ positions, int H, int G, int D,
                                                         int Dv, float scale_log2e, int window,
                                                         const float* __restrict__ sink, AT* __restrict__ out,
                                                         int64_t os, int64_t pairs) {
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
  const int Ck = G * D, Cv = G * Dv;
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
      const AT* kr = kc + ((int64_t)pages[j / PAGE] * PAGE + (j % PAGE)) * Ck + (int64_t)g * D;
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
                                hipStream_t st) {
  if (T <= 0 || d <= 0) return hipSuccess;
  if (S < 1 || S > SMAX) return hipErrorInvalidValue;
  auto a = [&](auto k) {
    k<<<(unsigned)T, NT, 0, st>>>(xs, s_stride, t_stride, y, ys, y_f32 != 0, y2, y2s, y2_f32 != 0, row_scale, mix, wr,
                                  rd, nw, eps, out, os, out_f32 != 0, total, ts, d);
  };
  switch (S) {
    case 1: a(stream_step_kernel<1>); break;
    case 2: a(stream_step_kernel<2>); break;
    case 3: a(stream_step_kernel<3>); break;
    case 4: a(stream_step_kernel<4>); break;
    case 5: a(stream_step_kernel<5>); break;
    case 6: a(stream_step_kernel<6>); break;
    case 7: a(stream_step_kernel<7>); break;
    default: a(stream_step_kernel<8>); break;
  }
  return hipGetLastError();
}

hipError_t kafka_hy_swish_clamp_mul(int f32, const void* gu, int64_t gs, void* out, int64_t os, int64_t T, int F,
                                    float limit, float alpha, hipStream_t st) {
  if (T <= 0 || F <= 0) return hipSuccess;
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
                                hipStream_t st) {
  if (T <= 0) return hipSuccess;
  if (D > WA_MAXD || Dv > 64 * WA_NV || G < 1 || H % G || window < 0) return hipErrorInvalidValue;
  const int64_t pairs = T * H;
  const int grid = (int)((pairs + NT / 64 - 1) / (NT / 64));
  DISPATCH_AT(f32, {
    window_attn_kernel<AT><<<grid, NT, 0, st>>>((const AT*)q, qs, (const AT*)kc, (const AT*)vt, bt, bt_stride, tok_seg,
                                                positions, H, G, D, Dv, scale * LOG2E, window, sink, (AT*)out, os,
                                                pairs);
  });
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
