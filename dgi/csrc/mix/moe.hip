// dgi/csrc/mix/moe.hip — mixture-of-experts feed-forward: routing, per-pair expert evaluation for
// small steps, and the combine of sorted-segment expert outputs for large ones.
//
//   moe_route         one wave per token: s = softmax(logits) over all R routes (fp32) or sigmoid of each, the
//                     `top` routes with the largest s + correction (ties: lowest index), weights = s of those;
//                     mode 2: the `top` largest logits, weights = softmax over those alone
//   silu_mul          silu(g) * u over fused [gate | up] rows
//   glu_rows          the expert activation with an optional per-row factor on gate and up first (a route
//                     weight on the expert's input, applied after the linear projections) and the clamped
//                     sigmoid-GLU form min(g, lim) sigmoid(alpha min(g, lim)) (clamp(u, +-lim) + 1)
//   moe_expert_gate_up / moe_expert_down   small steps: grid (expert, output tile), each workgroup walks the
//                     pairs that chose its expert straight from the stacked weights [E, 2 ff, W] / [E, W, ff]
//                     (see below); identity routes (e >= E) belong to no workgroup
//   moe_combine       out[t][w] = sum_k wt_k * ys[where[pair]][w]  (identity: wt_k * h[t][w]) + shared[t][w],
//                     the routes added in their fixed order k = 0..top-1; `where` maps a pair to its row in
//                     ys (null: the pair's own index), as the sorted segment GEMMs of a large step leave them
//
// Dot products run one output per wave with lanes striding the reduction dim, fp32 accumulation.
#include <algorithm>
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

// 16 bytes of weights as floats: 8 bf16 or 4 fp32
template <typename T> __device__ __forceinline__ void ld16(const T* p, float* f);
template <> __device__ __forceinline__ void ld16<uint16_t>(const uint16_t* p, float* f) {
  unpack8(*reinterpret_cast<const u32x4*>(p), f);
}
template <> __device__ __forceinline__ void ld16<float>(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}

// four consecutive weights as floats (8 bytes of bf16 or 16 of fp32): consecutive lanes then read
// consecutive 16-byte LDS words of the staged activations, which is bank-conflict free (eight-element
// chunks put lanes 32 bytes apart: an 8-way conflict)
template <typename T> __device__ __forceinline__ void ld4(const T* p, float* f);
template <> __device__ __forceinline__ void ld4<uint16_t>(const uint16_t* p, float* f) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
}
template <> __device__ __forceinline__ void ld4<float>(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}

constexpr int MAXR = 8;      // routes per lane: R <= 512

__global__ __launch_bounds__(64) void moe_route_kernel(int* __restrict__ idx, float* __restrict__ wts,
                                                       const float* __restrict__ logits, int l_stride,
                                                       const float* __restrict__ corr, int R, int top, int sigmoid) {
  __shared__ float wsel[64 * MAXR];      // the chosen routes' weights, in order of choice
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* lp = logits + (size_t)t * l_stride;
  float s[MAXR], c[MAXR];
  float m = -__builtin_inff();
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int r = lane + 64 * i;
    s[i] = r < R ? lp[r] : -__builtin_inff();
    m = fmaxf(m, s[i]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int r = lane + 64 * i;
    if (sigmoid == 1) s[i] = r < R ? 1.f / (1.f + expf(-s[i])) : 0.f;     // independent scores
    else s[i] = r < R ? expf(s[i] - m) : 0.f;
    sum += s[i];
  }
  const float inv = sigmoid == 1 ? 1.f : 1.f / wave_sum(sum);
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int r = lane + 64 * i;
    s[i] *= inv;
    c[i] = r < R ? s[i] + (corr ? corr[r] : 0.f) : -__builtin_inff();
  }
  if (sigmoid == 2) {
    // choice by the logits themselves, weights exp(z - max) over the chosen ones, normalised below; the first
    // pick is the row maximum, so every chosen term is exp of a non-positive number and the first is 1
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int r = lane + 64 * i;
      c[i] = r < R ? lp[r] : -__builtin_inff();
      s[i] = r < R ? expf(lp[r] - m) : 0.f;
    }
  }
  float chosen = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -__builtin_inff();
    int bi = 1 << 30;
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int r = lane + 64 * i;
      if (c[i] > bv) { bv = c[i]; bi = r; }          // ascending r within a lane: the lowest index wins ties
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      if (lane + 64 * i == bi) {
        idx[(size_t)t * top + k] = bi;
        wsel[k] = s[i];
        chosen += s[i];
        c[i] = -__builtin_inff();
      }
    }
  }
  chosen = wave_sum(chosen);              // each pick was added by the one lane that owns it
  __syncthreads();
  const float norm = sigmoid == 2 ? 1.f / chosen : 1.f;
  for (int k = lane; k < top; k += 64) wts[(size_t)t * top + k] = wsel[k] * norm;
}

template <typename T> __device__ __forceinline__ void st4(T* p, const float* f);
template <> __device__ __forceinline__ void st4<float>(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
}
template <> __device__ __forceinline__ void st4<uint16_t>(uint16_t* p, const float* f) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]));
}

// V = 4: four columns per thread (I, the row stride and the pointers allow 8 / 16-byte accesses)
template <typename T, int V>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int gu_stride, int rows, int I) {
  const size_t n = (size_t)rows * (I / V);
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const size_t r = i / (I / V), c = (i - r * (I / V)) * V;
    float g[V], u[V], o[V];
    if constexpr (V == 4) {
      ld4<T>(gu + r * gu_stride + c, g);
      ld4<T>(gu + r * gu_stride + I + c, u);
    } else {
      g[0] = ldf<T>(gu + r * gu_stride + c);
      u[0] = ldf<T>(gu + r * gu_stride + I + c);
    }
#pragma unroll
    for (int k = 0; k < V; ++k) o[k] = g[k] / (1.f + expf(-g[k])) * u[k];
    if constexpr (V == 4) st4<T>(out + r * I + c, o);
    else stf<T>(out + r * I + c, o[0]);
  }
}

// expert activation on fp32 pre-activations: kind 0 silu(g) * u; kind 1 the clamped sigmoid-GLU
__device__ __forceinline__ float expert_act(float g, float u, int kind, float limit, float alpha) {
  if (kind == 1) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.f + expf(-alpha * g)) * (u + 1.f);
  }
  return g / (1.f + expf(-g)) * u;
}

template <typename T, int V>
__global__ void glu_rows_kernel(T* __restrict__ out, const T* __restrict__ gu, int gu_stride, int rows, int I, int kind,
                                float limit, float alpha, const float* __restrict__ row_scale) {
  const size_t n = (size_t)rows * (I / V);
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const size_t r = i / (I / V), c = (i - r * (I / V)) * V;
    const float rs = row_scale ? row_scale[r] : 1.f;
    float g[V], u[V], o[V];
    if constexpr (V == 4) {
      ld4<T>(gu + r * gu_stride + c, g);
      ld4<T>(gu + r * gu_stride + I + c, u);
    } else {
      g[0] = ldf<T>(gu + r * gu_stride + c);
      u[0] = ldf<T>(gu + r * gu_stride + I + c);
    }
#pragma unroll
    for (int k = 0; k < V; ++k) o[k] = expert_act(g[k] * rs, u[k] * rs, kind, limit, alpha);
    if constexpr (V == 4) st4<T>(out + r * I + c, o);
    else stf<T>(out + r * I + c, o[0]);
  }
}

// ---------------------------------------------------------------------------------------------
// Expert-major evaluation for small steps: a workgroup owns (expert e, a tile of outputs) and walks
// the (token, route) pairs that chose e, PG at a time, so the expert's weight rows stream once per
// group of PG pairs (once in all for a decode step with a handful of tokens per expert) instead of
// once per pair.  The pairs of e are found by scanning idx and compacted into an LDS list (their
// order there does not matter: every pair's result is independent).
constexpr int CAP = 1024;    // pairs scanned per round
constexpr int OPB = 4;       // outputs per workgroup (1 per wave)

template <int PG>
__device__ __forceinline__ int collect_pairs(const int* __restrict__ idx, int base, int P, int e, int* list, int* cnt) {
  if (threadIdx.x == 0) *cnt = 0;
  __syncthreads();
  const int hi = min(P, base + CAP);
  for (int p = base + threadIdx.x; p < hi; p += blockDim.x)
    if (idx[p] == e) list[atomicAdd(cnt, 1)] = p;
  __syncthreads();
  return *cnt;
}

// mid[pair][f] = act(s Wg[e][f] . h_t, s Wu[e][f] . h_t), s = pair_scale[pair] (null: 1)     gate_up [E, 2 ff, W]
template <typename T, int PG>
__global__ __launch_bounds__(256) void moe_expert_gate_up_kernel(
    float* __restrict__ mid, const T* __restrict__ h, int h_stride, const int* __restrict__ idx,
    const T* __restrict__ gate_up, int P, int top, int ff, int W, const float* __restrict__ pair_scale, int act,
    float limit, float alpha) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  int* list = reinterpret_cast<int*>(sm);             // [CAP]
  T* hs = reinterpret_cast<T*>(sm + CAP);             // [PG][W] in the activation dtype (no rounding: h has it)
  __shared__ int cnt;
  const int e = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* wg = gate_up + (size_t)e * 2 * ff * W;
  for (int base = 0; base < P; base += CAP) {
    const int n = collect_pairs<PG>(idx, base, P, e, list, &cnt);
    for (int g0 = 0; g0 < n; g0 += PG) {
      const int np = min(PG, n - g0);
      __syncthreads();                                // the previous group's rows are fully read
      {
        constexpr int EV = 16 / sizeof(T);
        if (W % EV == 0 && h_stride % EV == 0 && ((uintptr_t)h & 15) == 0) {   // 16-byte copies, several in flight
          const int cpr = W / EV;
#pragma unroll 4
          for (int i = threadIdx.x; i < PG * cpr; i += 256) {
            const int p = i / cpr, c = i - p * cpr;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (p < np) v = *reinterpret_cast<const u32x4*>(h + (size_t)(list[g0 + p] / top) * h_stride + c * EV);
            *reinterpret_cast<u32x4*>(hs + (size_t)p * W + c * EV) = v;
          }
        } else {
          for (int i = threadIdx.x; i < PG * W; i += 256) {
            const int p = i / W, w = i - p * W;
            hs[i] = p < np ? h[(size_t)(list[g0 + p] / top) * h_stride + w] : T(0);
          }
        }
      }
      __syncthreads();
      for (int j = 0; j < OPB / 4; ++j) {
        const int f = blockIdx.y * OPB + wave * (OPB / 4) + j;
        if (f >= ff) break;
        const T* gp = wg + (size_t)f * W;
        const T* up = wg + (size_t)(ff + f) * W;
        float ag[PG], au[PG];
#pragma unroll
        for (int p = 0; p < PG; ++p) ag[p] = au[p] = 0.f;
        if (W % 4 == 0 && ((uintptr_t)gate_up & 15) == 0) {
#pragma unroll 8
          for (int c = lane; c < W / 4; c += 64) {
            float a[4], b[4];
            ld4<T>(gp + c * 4, a);
            ld4<T>(up + c * 4, b);
#pragma unroll
            for (int p = 0; p < PG; ++p) {
              float x[4];
              ld4<T>(hs + p * W + c * 4, x);
              ag[p] += a[0] * x[0] + a[1] * x[1] + a[2] * x[2] + a[3] * x[3];
              au[p] += b[0] * x[0] + b[1] * x[1] + b[2] * x[2] + b[3] * x[3];
            }
          }
        } else {
          for (int w = lane; w < W; w += 64) {
            const float a = ldf<T>(gp + w), b = ldf<T>(up + w);
#pragma unroll
            for (int p = 0; p < PG; ++p) {
              const float x = ldf<T>(hs + p * W + w);
              ag[p] += a * x;
              au[p] += b * x;
            }
          }
        }
#pragma unroll
        for (int p = 0; p < PG; ++p) {
          const float sg = wave_sum(ag[p]), su = wave_sum(au[p]);
          if (lane == 0 && p < np) {
            const int pair = list[g0 + p];
            const float ps = pair_scale ? pair_scale[pair] : 1.f;
            mid[(size_t)pair * ff + f] = expert_act(sg * ps, su * ps, act, limit, alpha);
          }
        }
      }
    }
    __syncthreads();                                  // list is rebuilt by the next round
  }
}

// ys[pair][w] = Wd[e][w] . mid[pair]                           down [E, W, ff]
template <typename T, int PG>
__global__ __launch_bounds__(256) void moe_expert_down_kernel(
    T* __restrict__ ys, const float* __restrict__ mid, const int* __restrict__ idx, const T* __restrict__ down, int P,
    int ff, int W) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  int* list = reinterpret_cast<int*>(sm);             // [CAP]
  float* ms = sm + CAP;                               // [PG][ff]
  __shared__ int cnt;
  const int e = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int base = 0; base < P; base += CAP) {
    const int n = collect_pairs<PG>(idx, base, P, e, list, &cnt);
    for (int g0 = 0; g0 < n; g0 += PG) {
      const int np = min(PG, n - g0);
      __syncthreads();
      if (ff % 4 == 0) {
        const int cpr = ff / 4;
#pragma unroll 4
        for (int i = threadIdx.x; i < PG * cpr; i += 256) {
          const int p = i / cpr, c = i - p * cpr;
          float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
          if (p < np) v = *reinterpret_cast<const float4*>(mid + (size_t)list[g0 + p] * ff + c * 4);
          *reinterpret_cast<float4*>(ms + (size_t)p * ff + c * 4) = v;
        }
      } else {
        for (int i = threadIdx.x; i < PG * ff; i += 256) {
          const int p = i / ff, f = i - p * ff;
          ms[i] = p < np ? mid[(size_t)list[g0 + p] * ff + f] : 0.f;
        }
      }
      __syncthreads();
      for (int j = 0; j < OPB / 4; ++j) {
        const int w = blockIdx.y * OPB + wave * (OPB / 4) + j;
        if (w >= W) break;
        const T* dp = down + ((size_t)e * W + w) * ff;
        float acc[PG];
#pragma unroll
        for (int p = 0; p < PG; ++p) acc[p] = 0.f;
        if (ff % 4 == 0 && ((uintptr_t)down & 15) == 0) {
#pragma unroll 4
          for (int c = lane; c < ff / 4; c += 64) {
            float a[4];
            ld4<T>(dp + c * 4, a);
#pragma unroll
            for (int p = 0; p < PG; ++p) {
              const float4 x = *reinterpret_cast<const float4*>(ms + p * ff + c * 4);
              acc[p] += a[0] * x.x + a[1] * x.y + a[2] * x.z + a[3] * x.w;
            }
          }
        } else {
          for (int f = lane; f < ff; f += 64) {
            const float a = ldf<T>(dp + f);
#pragma unroll
            for (int p = 0; p < PG; ++p) acc[p] += a * ms[p * ff + f];
          }
        }
#pragma unroll
        for (int p = 0; p < PG; ++p) {
          const float sd = wave_sum(acc[p]);
          if (lane == 0 && p < np) stf<T>(ys + (size_t)list[g0 + p] * W + w, sd);
        }
      }
    }
    __syncthreads();
  }
}

template <typename T, int V>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    T* __restrict__ out, const T* __restrict__ ys, const int* __restrict__ where, const T* __restrict__ h, int h_stride,
    const int* __restrict__ idx, const float* __restrict__ wts, const T* __restrict__ shared, int shared_stride, int E,
    int top, int W) {
  const int t = blockIdx.x;
  const int w = (blockIdx.y * 256 + threadIdx.x) * V;
  if (w >= W) return;
  float acc[V], v[V];
#pragma unroll
  for (int k = 0; k < V; ++k) acc[k] = 0.f;
  if (shared) {
    if constexpr (V == 4) ld4<T>(shared + (size_t)t * shared_stride + w, acc);
    else acc[0] = ldf<T>(shared + (size_t)t * shared_stride + w);
  }
  for (int k = 0; k < top; ++k) {
    const int e = idx[(size_t)t * top + k];
    const float wt = wts ? wts[(size_t)t * top + k] : 1.f;
    const T* src = (e >= E || e < 0) ? h + (size_t)t * h_stride + w
                                     : ys + (size_t)(where ? where[(size_t)t * top + k] : t * top + k) * W + w;
    if constexpr (V == 4) ld4<T>(src, v);
    else v[0] = ldf<T>(src);
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] += wt * v[j];
  }
  if constexpr (V == 4) st4<T>(out + (size_t)t * W + w, acc);
  else stf<T>(out + (size_t)t * W + w, acc[0]);
}

}  // namespace

extern "C" int dgi_moe_route(int* idx, float* wts, const float* logits, int l_stride, const float* corr, int T, int R,
                             int top, int sigmoid, hipStream_t s) {
  if (T == 0) return 0;
  if (R > 64 * MAXR || top > R || top < 1) return -2;
  moe_route_kernel<<<T, 64, 0, s>>>(idx, wts, logits, l_stride, corr, R, top, sigmoid);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_glu_silu(void* out, const void* gu, int gu_stride, int rows, int I, int is_f32, hipStream_t s) {
  if (rows == 0 || I == 0) return 0;
  const bool vec = I % 4 == 0 && gu_stride % 4 == 0 && (((uintptr_t)out | (uintptr_t)gu) & 15) == 0;
  const size_t n = (size_t)rows * (vec ? I / 4 : I);
  const int blocks = (int)((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256);
  if (is_f32) {
    if (vec) silu_mul_kernel<float, 4><<<blocks, 256, 0, s>>>((float*)out, (const float*)gu, gu_stride, rows, I);
    else silu_mul_kernel<float, 1><<<blocks, 256, 0, s>>>((float*)out, (const float*)gu, gu_stride, rows, I);
  } else {
    if (vec) silu_mul_kernel<uint16_t, 4><<<blocks, 256, 0, s>>>((uint16_t*)out, (const uint16_t*)gu, gu_stride, rows, I);
    else silu_mul_kernel<uint16_t, 1><<<blocks, 256, 0, s>>>((uint16_t*)out, (const uint16_t*)gu, gu_stride, rows, I);
  }
  DGI_CHECK_LAUNCH();
  return 0;
}

// pairs per group by LDS budget: PG rows of `row_bytes` + the pair list within 96 KiB (two workgroups a CU)
static int pick_pg(size_t row_bytes) {
  const size_t room = 96 * 1024 - CAP * 4;
  return row_bytes * 8 <= room ? 8 : (row_bytes * 4 <= room ? 4 : (row_bytes * 2 <= room ? 2 : (row_bytes <= room ? 1 : 0)));
}

// more than 64 KiB of dynamic LDS has to be allowed per kernel, once
template <typename K>
static int allow_lds(K kernel, size_t lds) {
  if (lds <= 64 * 1024) return 0;
  return (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
}

extern "C" int dgi_glu_rows(void* out, const void* gu, int gu_stride, int rows, int I, int kind, float limit, float alpha,
                            const float* row_scale, int is_f32, hipStream_t s) {
  if (rows == 0 || I == 0) return 0;
  const bool vec = I % 4 == 0 && gu_stride % 4 == 0 && (((uintptr_t)out | (uintptr_t)gu) & 15) == 0;
  const size_t n = (size_t)rows * (vec ? I / 4 : I);
  const int blocks = (int)((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256);
#define DGI_GR(TT_, VV_) \
  glu_rows_kernel<TT_, VV_><<<blocks, 256, 0, s>>>((TT_*)out, (const TT_*)gu, gu_stride, rows, I, kind, limit, alpha, row_scale)
  if (is_f32) { if (vec) DGI_GR(float, 4); else DGI_GR(float, 1); }
  else { if (vec) DGI_GR(uint16_t, 4); else DGI_GR(uint16_t, 1); }
#undef DGI_GR
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_moe_expert_gate_up(float* mid, const void* h, int h_stride, const int* idx, const void* gate_up,
                                      int T, int E, int top, int ff, int W, const float* pair_scale, int act, float limit,
                                      float alpha, int is_f32, hipStream_t s) {
  if (T == 0 || E == 0) return 0;
  const size_t es = is_f32 ? 4 : 2;
  const int pg = pick_pg((size_t)W * es);
  if (!pg) return -2;
  const dim3 grid(E, (ff + OPB - 1) / OPB);
  if (grid.y > 65535) return -3;
  const size_t lds = (size_t)pg * W * es + CAP * 4;
#define DGI_GU(TT_, PG_)                                                                                        \
  do {                                                                                                          \
    static const int ok = allow_lds(moe_expert_gate_up_kernel<TT_, PG_>, 96 * 1024);                            \
    if (ok != 0) return ok;                                                                                     \
    moe_expert_gate_up_kernel<TT_, PG_><<<grid, 256, lds, s>>>(mid, (const TT_*)h, h_stride, idx, (const TT_*)gate_up, \
                                                              T * top, top, ff, W, pair_scale, act, limit, alpha); \
  } while (0)
  if (is_f32) { if (pg == 8) DGI_GU(float, 8); else if (pg == 4) DGI_GU(float, 4); else if (pg == 2) DGI_GU(float, 2); else DGI_GU(float, 1); }
  else { if (pg == 8) DGI_GU(uint16_t, 8); else if (pg == 4) DGI_GU(uint16_t, 4); else if (pg == 2) DGI_GU(uint16_t, 2); else DGI_GU(uint16_t, 1); }
#undef DGI_GU
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_moe_expert_down(void* ys, const float* mid, const int* idx, const void* down, int T, int E, int top,
                                   int ff, int W, int is_f32, hipStream_t s) {
  if (T == 0 || E == 0) return 0;
  const int pg = pick_pg((size_t)ff * 4);
  if (!pg) return -2;
  const dim3 grid(E, (W + OPB - 1) / OPB);
  if (grid.y > 65535) return -3;
  const size_t lds = ((size_t)pg * ff + CAP) * 4;
#define DGI_DN(TT_, PG_)                                                                                         \
  do {                                                                                                           \
    static const int ok = allow_lds(moe_expert_down_kernel<TT_, PG_>, 96 * 1024);                                \
    if (ok != 0) return ok;                                                                                      \
    moe_expert_down_kernel<TT_, PG_><<<grid, 256, lds, s>>>((TT_*)ys, mid, idx, (const TT_*)down, T * top, ff, W); \
  } while (0)
  if (is_f32) { if (pg == 8) DGI_DN(float, 8); else if (pg == 4) DGI_DN(float, 4); else if (pg == 2) DGI_DN(float, 2); else DGI_DN(float, 1); }
  else { if (pg == 8) DGI_DN(uint16_t, 8); else if (pg == 4) DGI_DN(uint16_t, 4); else if (pg == 2) DGI_DN(uint16_t, 2); else DGI_DN(uint16_t, 1); }
#undef DGI_DN
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_moe_combine(void* out, const void* ys, const int* where, const void* h, int h_stride, const int* idx,
                               const float* wts, const void* shared, int shared_stride, int T, int E, int top, int W,
                               int is_f32, hipStream_t s) {
  if (T == 0) return 0;
  const bool vec = W % 4 == 0 && h_stride % 4 == 0 && shared_stride % 4 == 0 &&
                   (((uintptr_t)out | (uintptr_t)ys | (uintptr_t)h | (uintptr_t)shared) & 15) == 0;
  const dim3 grid(T, vec ? (W / 4 + 255) / 256 : (W + 255) / 256);
  if (grid.y > 65535) return -3;
#define DGI_COMB(TT_, VV_)                                                                                          \
  moe_combine_kernel<TT_, VV_><<<grid, 256, 0, s>>>((TT_*)out, (const TT_*)ys, where, (const TT_*)h, h_stride, idx, wts, \
                                                    (const TT_*)shared, shared_stride, E, top, W)
  if (is_f32) { if (vec) DGI_COMB(float, 4); else DGI_COMB(float, 1); }
  else { if (vec) DGI_COMB(uint16_t, 4); else DGI_COMB(uint16_t, 1); }
#undef DGI_COMB
  DGI_CHECK_LAUNCH();
  return 0;
}
