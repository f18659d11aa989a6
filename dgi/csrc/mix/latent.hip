// dgi/csrc/mix/latent.hip — row kernels of latent-attention models on an fp32 residual stream.
//
//   stream_add_norm   x += y   (or x += y / rms(y) * post_w; or x += y + y2, two sublayers of one step)   and
//                     out = x / rms(x) * next_w  (or out = x)
//                     in one pass over the row: the residual add of one sublayer fused with the RMS
//                     norm that feeds the next GEMM (the fused_add_rmsnorm of models whose stream is fp32)
//   latent_prep       row = [query latent | key/value latent | key part | ...] from one fused GEMM:
//                     RMS norm + weight of the query latent -> cq; RMS norm + weight of the key/value
//                     latent and rotary of the key part -> one cache row [c | r] in the paged pool
//   rotate_heads      rotary on `dims` entries at a fixed offset inside every head of a row, in place
//   gate_heads        [H, T, dv] head outputs -> [T, H * dv] times sigmoid(gate), one gate per head or per element
//   gelu_tanh         tanh-form GELU, optionally times a slice of a table row gathered by token id
//
// rms(v) = sqrt(mean(v^2) + eps).  Everything is computed in fp32; activations are bf16 or fp32.
// One 256-thread workgroup per row, the row held in registers between the reduction and the store.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

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
template <typename T> __device__ __forceinline__ void st4(T* p, const float* f);
template <> __device__ __forceinline__ void st4<float>(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
}
template <> __device__ __forceinline__ void st4<uint16_t>(uint16_t* p, const float* f) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]));
}

constexpr int NT = 256;          // threads per row
constexpr int MAXV = 8;          // 4-column chunks per thread: rows up to NT * 4 * MAXV = 8192 columns

// sum over the workgroup (all threads get it); `red` is NT / 64 floats of LDS, reusable after the call
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();                                   // earlier readers of red are done
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) s += red[i];
  return s;
}

// V = 4: 16-byte accesses (W, strides and pointers allow them); V = 1: any shape
template <typename TY, typename TO, int V>
__global__ __launch_bounds__(NT) void stream_add_norm_kernel(float* __restrict__ x, int W, const TY* __restrict__ y,
                                                             int y_stride, const float* __restrict__ post_w,
                                                             const float* __restrict__ next_w, float eps,
                                                             TO* __restrict__ out, const void* __restrict__ y2,
                                                             int y2_stride, int y2_f32) {
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  float* xr = x + (size_t)row * W;
  const TY* yr = y ? y + (size_t)row * y_stride : nullptr;
  // second addend of the same step (bf16 or fp32, chosen at run time: uniform branches)
  const float* y2f = (y2 && y2_f32) ? (const float*)y2 + (size_t)row * y2_stride : nullptr;
  const uint16_t* y2h = (y2 && !y2_f32) ? (const uint16_t*)y2 + (size_t)row * y2_stride : nullptr;
  float xv[MAXV][V], yv[MAXV][V];
  float ssy = 0.f;
#pragma unroll
  for (int k = 0; k < MAXV; ++k) {
    const int c = (threadIdx.x + k * NT) * V;
    if (c < W) {
      if constexpr (V == 4) {
        ld4<float>(xr + c, xv[k]);
        if (yr) ld4<TY>(yr + c, yv[k]);
      } else {
        xv[k][0] = xr[c];
        if (yr) yv[k][0] = ldf<TY>(yr + c);
      }
      if (yr) {
#pragma unroll
        for (int j = 0; j < V; ++j) ssy += yv[k][j] * yv[k][j];
      }
    }
  }
  if (yr) {
    float inv_y = 1.f;
    if (post_w) inv_y = 1.f / sqrtf(block_sum(ssy, red) / (float)W + eps);
#pragma unroll
    for (int k = 0; k < MAXV; ++k) {
      const int c = (threadIdx.x + k * NT) * V;
      if (c < W) {
#pragma unroll
        for (int j = 0; j < V; ++j) yv[k][j] = post_w ? yv[k][j] * inv_y * post_w[c + j] : yv[k][j];
        if (y2f || y2h) {
          float zv[V];
          if constexpr (V == 4) {
            if (y2f) ld4<float>(y2f + c, zv); else ld4<uint16_t>(y2h + c, zv);
          } else {
            zv[0] = y2f ? y2f[c] : bf16_to_f32(y2h[c]);
          }
#pragma unroll
          for (int j = 0; j < V; ++j) yv[k][j] += zv[j];
        }
#pragma unroll
        for (int j = 0; j < V; ++j) xv[k][j] += yv[k][j];
        if constexpr (V == 4) st4<float>(xr + c, xv[k]);
        else xr[c] = xv[k][0];
      }
    }
  }
  if (!out) return;
  TO* orow = out + (size_t)row * W;
  float inv_x = 1.f;
  if (next_w) {
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < MAXV; ++k) {
      const int c = (threadIdx.x + k * NT) * V;
      if (c < W) {
#pragma unroll
        for (int j = 0; j < V; ++j) ss += xv[k][j] * xv[k][j];
      }
    }
    inv_x = 1.f / sqrtf(block_sum(ss, red) / (float)W + eps);
  }
#pragma unroll
  for (int k = 0; k < MAXV; ++k) {
    const int c = (threadIdx.x + k * NT) * V;
    if (c < W) {
      float o[V];
#pragma unroll
      for (int j = 0; j < V; ++j) o[j] = next_w ? xv[k][j] * inv_x * next_w[c + j] : xv[k][j];
      if constexpr (V == 4) st4<TO>(orow + c, o);
      else stf<TO>(orow + c, o[0]);
    }
  }
}

// One workgroup per row.  Query latent: columns [0, q_rank); key/value latent [q_rank, q_rank + kv_rank);
// key part [q_rank + kv_rank, q_rank + kv_rank + rot_dim), of which the first `dims` rotate.
template <typename T, bool VEC>
__global__ __launch_bounds__(NT) void latent_prep_kernel(const T* __restrict__ proj, int stride, int q_rank, int kv_rank,
                                                         int rot_dim, const float* __restrict__ dq_w,
                                                         const float* __restrict__ dkv_w, float eps,
                                                         const int* __restrict__ positions, const int* __restrict__ slots,
                                                         const float* __restrict__ cos_sin, int dims, int interleaved,
                                                         T* __restrict__ cq, T* __restrict__ cache) {
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  const T* p = proj + (size_t)row * stride;
  // RMS norm of n values at src times w -> dst; VEC: 16-byte chunks held in registers between the sum and the store
  auto norm_part = [&](const T* src, int n, const float* w, T* dst) {
    constexpr int E = 16 / sizeof(T);
    if (VEC) {
      float v[2][8];
      float ss = 0.f;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int c = (threadIdx.x + k * NT) * E;
        if (c < n) {
          const uint4 raw = *reinterpret_cast<const uint4*>(src + c);
          if constexpr (sizeof(T) == 2) unpack8(__builtin_bit_cast(u32x4, raw), v[k]);
          else { v[k][0] = __uint_as_float(raw.x); v[k][1] = __uint_as_float(raw.y); v[k][2] = __uint_as_float(raw.z); v[k][3] = __uint_as_float(raw.w); }
#pragma unroll
          for (int j = 0; j < E; ++j) ss += v[k][j] * v[k][j];
        }
      }
      const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int c = (threadIdx.x + k * NT) * E;
        if (c < n) {
#pragma unroll
          for (int j = 0; j < E; ++j) v[k][j] *= inv * w[c + j];
          uint4 o;
          if constexpr (sizeof(T) == 2) o = __builtin_bit_cast(uint4, pack8(v[k]));
          else o = make_uint4(__float_as_uint(v[k][0]), __float_as_uint(v[k][1]), __float_as_uint(v[k][2]), __float_as_uint(v[k][3]));
          *reinterpret_cast<uint4*>(dst + c) = o;
        }
      }
    } else {
      float ss = 0.f;
      for (int c = threadIdx.x; c < n; c += NT) {
        const float x = ldf<T>(src + c);
        ss += x * x;
      }
      const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
      for (int c = threadIdx.x; c < n; c += NT) stf<T>(dst + c, ldf<T>(src + c) * inv * w[c]);
    }
  };
  norm_part(p, q_rank, dq_w, cq + (size_t)row * q_rank);
  if (!cache) return;
  const int slot = slots[row];
  if (slot < 0) return;                               // uniform over the workgroup
  T* dst = cache + (size_t)slot * (kv_rank + rot_dim);
  const T* lat = p + q_rank;
  norm_part(lat, kv_rank, dkv_w, dst);
  const T* kp = lat + kv_rank;
  T* kd = dst + kv_rank;
  const int half = dims >> 1;
  const float* cs = cos_sin ? cos_sin + (size_t)positions[row] * dims : nullptr;
  for (int i = threadIdx.x; i < half; i += NT) {
    const int i0 = interleaved ? 2 * i : i, i1 = interleaved ? 2 * i + 1 : i + half;
    const float u = ldf<T>(kp + i0), v = ldf<T>(kp + i1);
    const float c = cs[i], s = cs[half + i];
    stf<T>(kd + i0, u * c - v * s);
    stf<T>(kd + i1, v * c + u * s);
  }
  for (int c = dims + threadIdx.x; c < rot_dim; c += NT) kd[c] = kp[c];
}

// x[t][h * hs + off + (pair)] rotated by the row's position; grid (T), threads over H * dims / 2 pairs
template <typename T>
__global__ __launch_bounds__(NT) void rotate_heads_kernel(T* __restrict__ x, int stride, const int* __restrict__ positions,
                                                          const float* __restrict__ cos_sin, int dims, int interleaved,
                                                          int H, int hs, int off) {
  const int t = blockIdx.x, half = dims >> 1;
  const float* cs = cos_sin + (size_t)positions[t] * dims;
  T* row = x + (size_t)t * stride;
  for (int i = threadIdx.x; i < H * half; i += NT) {
    const int h = i / half, k = i - h * half;
    T* p = row + (size_t)h * hs + off;
    const int i0 = interleaved ? 2 * k : k, i1 = interleaved ? 2 * k + 1 : k + half;
    const float u = ldf<T>(p + i0), v = ldf<T>(p + i1);
    const float c = cs[k], sn = cs[half + k];
    stf<T>(p + i0, u * c - v * sn);
    stf<T>(p + i1, v * c + u * sn);
  }
}

// out[t][h * dv + d] = ov[h][t][d] * sigmoid(gate[t][h] or gate[t][h * dv + d]); grid (T, ceil(H * dv / 256))
template <typename T>
__global__ __launch_bounds__(NT) void gate_heads_kernel(T* __restrict__ out, const T* __restrict__ ov, long long ov_hs,
                                                        long long ov_ts, const T* __restrict__ gate, int gate_stride,
                                                        int per_head, int H, int dv) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * NT + threadIdx.x;
  if (c >= H * dv) return;
  const int h = c / dv, d = c - h * dv;
  float v = ldf<T>(ov + (size_t)h * ov_hs + (size_t)t * ov_ts + d);
  if (gate) v *= 1.f / (1.f + expf(-ldf<T>(gate + (size_t)t * gate_stride + (per_head ? h : c))));
  stf<T>(out + (size_t)t * H * dv + c, v);
}

// tanh(a) = sign(a) (1 - e) / (1 + e), e = exp(-2 |a|), through the hardware exp / rcp (absolute error below 2e-7)
// eight (bf16) / four (fp32) consecutive value dims per thread: dv, the strides and the pointers allow 16-byte accesses
template <typename T>
__global__ __launch_bounds__(NT) void gate_heads_vec_kernel(T* __restrict__ out, const T* __restrict__ ov, long long ov_hs,
                                                            long long ov_ts, const T* __restrict__ gate, int gate_stride,
                                                            int per_head, int H, int dv) {
  constexpr int E = 16 / sizeof(T);
  const int t = blockIdx.x;
  const int c = (blockIdx.y * NT + threadIdx.x) * E;
  if (c >= H * dv) return;
  const int h = c / dv, d = c - h * dv;
  const uint4 raw = *reinterpret_cast<const uint4*>(ov + (size_t)h * ov_hs + (size_t)t * ov_ts + d);
  float v[8], g[8];
  if constexpr (sizeof(T) == 2) unpack8(__builtin_bit_cast(u32x4, raw), v);
  else { v[0] = __uint_as_float(raw.x); v[1] = __uint_as_float(raw.y); v[2] = __uint_as_float(raw.z); v[3] = __uint_as_float(raw.w); }
  if (gate) {
    if (per_head) {
      const float s = 1.f / (1.f + expf(-ldf<T>(gate + (size_t)t * gate_stride + h)));
#pragma unroll
      for (int j = 0; j < E; ++j) v[j] *= s;
    } else {
      const uint4 gr = *reinterpret_cast<const uint4*>(gate + (size_t)t * gate_stride + c);
      if constexpr (sizeof(T) == 2) unpack8(__builtin_bit_cast(u32x4, gr), g);
      else { g[0] = __uint_as_float(gr.x); g[1] = __uint_as_float(gr.y); g[2] = __uint_as_float(gr.z); g[3] = __uint_as_float(gr.w); }
#pragma unroll
      for (int j = 0; j < E; ++j) v[j] *= 1.f / (1.f + expf(-g[j]));
    }
  }
  uint4 o;
  if constexpr (sizeof(T) == 2) o = __builtin_bit_cast(uint4, pack8(v));
  else o = make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3]));
  *reinterpret_cast<uint4*>(out + (size_t)t * H * dv + c) = o;
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  const float a = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  const float e = __expf(-2.f * fabsf(a));
  const float t = copysignf((1.f - e) * __builtin_amdgcn_rcpf(1.f + e), a);
  return 0.5f * z * (1.f + t);
}

// out[t][c] = gelu(x[t][c]) (* table[ids[t]][col0 + c]); grid-stride over T * n
template <typename T>
__global__ __launch_bounds__(NT) void gelu_tanh_kernel(T* __restrict__ out, const T* __restrict__ x, int x_stride, int rows,
                                                       int n, const T* __restrict__ table, int t_stride, int vocab,
                                                       const int* __restrict__ ids, int col0) {
  const size_t total = (size_t)rows * n;
  for (size_t i = (size_t)blockIdx.x * NT + threadIdx.x; i < total; i += (size_t)gridDim.x * NT) {
    const size_t r = i / n;
    const int c = (int)(i - r * n);
    float v = gelu_tanh_f(ldf<T>(x + r * x_stride + c));
    if (table) {
      const int id = min(max(ids[r], 0), vocab - 1);    // no read outside the table
      v *= ldf<T>(table + (size_t)id * t_stride + col0 + c);
    }
    stf<T>(out + i, v);
  }
}

template <typename T, int V>
__global__ __launch_bounds__(NT) void gelu_tanh_vec_kernel(T* __restrict__ out, const T* __restrict__ x, int x_stride,
                                                           int rows, int n) {
  const size_t total = (size_t)rows * (n / V);
  for (size_t i = (size_t)blockIdx.x * NT + threadIdx.x; i < total; i += (size_t)gridDim.x * NT) {
    const size_t r = i / (n / V);
    const int c = (int)(i - r * (n / V)) * V;
    float v[V];
    ld4<T>(x + r * x_stride + c, v);
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] = gelu_tanh_f(v[j]);
    st4<T>(out + r * n + c, v);
  }
}

}  // namespace

extern "C" int dgi_stream_add_norm(float* x, int T, int W, const void* y, int y_stride, int y_f32, const float* post_w,
                                   const float* next_w, float eps, void* out, int out_f32, const void* y2, int y2_stride,
                                   int y2_f32, hipStream_t s) {
  if (T == 0 || W == 0) return 0;
  if (W > NT * 4 * MAXV) return -3;
  if (y2 && !y) return -5;
  const bool vec = W % 4 == 0 && y_stride % 4 == 0 && y2_stride % 4 == 0 &&
                   (((uintptr_t)x | (uintptr_t)y | (uintptr_t)out | (uintptr_t)y2) & 15) == 0 &&
                   W >= NT * 4;       // narrow rows: one column per thread and chunk keeps every thread busy
#define DGI_SAN(TY_, TO_)                                                                                              \
  do {                                                                                                                 \
    if (vec) stream_add_norm_kernel<TY_, TO_, 4><<<T, NT, 0, s>>>(x, W, (const TY_*)y, y_stride, post_w, next_w, eps, (TO_*)out, y2, y2_stride, y2_f32); \
    else if (W <= NT * MAXV) stream_add_norm_kernel<TY_, TO_, 1><<<T, NT, 0, s>>>(x, W, (const TY_*)y, y_stride, post_w, next_w, eps, (TO_*)out, y2, y2_stride, y2_f32); \
    else return -4;                                                                                                    \
  } while (0)
  if (y_f32) { if (out_f32) DGI_SAN(float, float); else DGI_SAN(float, uint16_t); }
  else { if (out_f32) DGI_SAN(uint16_t, float); else DGI_SAN(uint16_t, uint16_t); }
#undef DGI_SAN
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_latent_prep(const void* proj, int stride, int is_f32, int T, int q_rank, int kv_rank, int rot_dim,
                               const float* dq_w, const float* dkv_w, float eps, const int* positions, const int* slots,
                               const float* cos_sin, int dims, int interleaved, void* cq, void* cache, hipStream_t s) {
  if (T == 0) return 0;
  if (q_rank <= 0) return -2;
  if (cache && (kv_rank <= 0 || rot_dim < 0 || dims > rot_dim || (dims & 1) || (dims > 0 && !cos_sin) || !dkv_w || !slots))
    return -3;
  // 16-byte accesses: both latents and every row / cache start are multiples of the chunk, at most two chunks a thread
  const int E = is_f32 ? 4 : 8;
  const bool vec = q_rank % E == 0 && stride % E == 0 && q_rank <= 2 * NT * E && (((uintptr_t)proj | (uintptr_t)cq) & 15) == 0 &&
                   (!cache || (kv_rank % E == 0 && (kv_rank + rot_dim) % E == 0 && kv_rank <= 2 * NT * E && ((uintptr_t)cache & 15) == 0));
#define DGI_LP(TT_, VV_)                                                                                                  \
  latent_prep_kernel<TT_, VV_><<<T, NT, 0, s>>>((const TT_*)proj, stride, q_rank, kv_rank, rot_dim, dq_w, dkv_w, eps, positions, \
                                               slots, cos_sin, dims, interleaved, (TT_*)cq, (TT_*)cache)
  if (is_f32) { if (vec) DGI_LP(float, true); else DGI_LP(float, false); }
  else { if (vec) DGI_LP(uint16_t, true); else DGI_LP(uint16_t, false); }
#undef DGI_LP
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_rotate_heads(void* x, int stride, int is_f32, int T, const int* positions, const float* cos_sin, int dims,
                                int interleaved, int H, int hs, int off, hipStream_t s) {
  if (T == 0 || dims == 0 || H == 0) return 0;
  if ((dims & 1) || off < 0 || off + dims > hs || (long long)H * hs > stride) return -2;
  if (is_f32) rotate_heads_kernel<float><<<T, NT, 0, s>>>((float*)x, stride, positions, cos_sin, dims, interleaved, H, hs, off);
  else rotate_heads_kernel<uint16_t><<<T, NT, 0, s>>>((uint16_t*)x, stride, positions, cos_sin, dims, interleaved, H, hs, off);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_gate_heads(void* out, const void* ov, long long ov_hs, long long ov_ts, const void* gate,
                              int gate_stride, int per_head, int T, int H, int dv, int is_f32, hipStream_t s) {
  if (T == 0 || H * dv == 0) return 0;
  {
    const int E = is_f32 ? 4 : 8;
    const bool galign = !gate || per_head || (gate_stride % E == 0 && ((uintptr_t)gate & 15) == 0);
    if (dv % E == 0 && ov_hs % E == 0 && ov_ts % E == 0 && (((uintptr_t)out | (uintptr_t)ov) & 15) == 0 && galign) {
      const dim3 vgrid(T, (H * dv / E + NT - 1) / NT);
      if (vgrid.y > 65535) return -3;
      if (is_f32)
        gate_heads_vec_kernel<float><<<vgrid, NT, 0, s>>>((float*)out, (const float*)ov, ov_hs, ov_ts, (const float*)gate,
                                                         gate_stride, per_head, H, dv);
      else
        gate_heads_vec_kernel<uint16_t><<<vgrid, NT, 0, s>>>((uint16_t*)out, (const uint16_t*)ov, ov_hs, ov_ts,
                                                            (const uint16_t*)gate, gate_stride, per_head, H, dv);
      DGI_CHECK_LAUNCH();
      return 0;
    }
  }
  const dim3 grid(T, (H * dv + NT - 1) / NT);
  if (grid.y > 65535) return -3;
  if (is_f32)
    gate_heads_kernel<float><<<grid, NT, 0, s>>>((float*)out, (const float*)ov, ov_hs, ov_ts, (const float*)gate,
                                                 gate_stride, per_head, H, dv);
  else
    gate_heads_kernel<uint16_t><<<grid, NT, 0, s>>>((uint16_t*)out, (const uint16_t*)ov, ov_hs, ov_ts,
                                                    (const uint16_t*)gate, gate_stride, per_head, H, dv);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_gelu_tanh(void* out, const void* x, int x_stride, int rows, int n, const void* table, int t_stride,
                             int vocab, const int* ids, int col0, int is_f32, hipStream_t s) {
  if (rows == 0 || n == 0) return 0;
  const bool vec = !table && n % 4 == 0 && x_stride % 4 == 0 && (((uintptr_t)out | (uintptr_t)x) & 15) == 0;
  const size_t total = (size_t)rows * (vec ? n / 4 : n);
  const int blocks = (int)((total + NT - 1) / NT > 65535 * 4 ? 65535 * 4 : (total + NT - 1) / NT);
  if (is_f32) {
    if (vec) gelu_tanh_vec_kernel<float, 4><<<blocks, NT, 0, s>>>((float*)out, (const float*)x, x_stride, rows, n);
    else gelu_tanh_kernel<float><<<blocks, NT, 0, s>>>((float*)out, (const float*)x, x_stride, rows, n, (const float*)table,
                                                       t_stride, vocab, ids, col0);
  } else {
    if (vec) gelu_tanh_vec_kernel<uint16_t, 4><<<blocks, NT, 0, s>>>((uint16_t*)out, (const uint16_t*)x, x_stride, rows, n);
    else gelu_tanh_kernel<uint16_t><<<blocks, NT, 0, s>>>((uint16_t*)out, (const uint16_t*)x, x_stride, rows, n,
                                                          (const uint16_t*)table, t_stride, vocab, ids, col0);
  }
  DGI_CHECK_LAUNCH();
  return 0;
}
