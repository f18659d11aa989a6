// dgi/csrc/mix/qk_prep.hip — q / k RMS norm, rotary positions and the paged K/V write for mixers whose
// norm runs over the WHOLE q (and the whole k) projection of a token, or whose rotary pairs are the halves
// (i, i + rd/2) of a head; qknorm_rope_cache.hip is the per-head, interleaved-pair form of the same step.
//
// One workgroup per token reads its fused projection row [q: H*dk | k: G*dk | v: G*dv | ...] and
//   * replaces q by  rot(q / rms * qw)  in place,
//   * writes  rot(k / rms * kw)  and v into the paged cache at the row's slot,
// with rms = sqrt(mean(x^2) + eps) over the head (qw / kw [dk]) or, `full`, over the whole projection
// (qw [H*dk], kw [G*dk]).  rot() turns pairs of the first rd dims of every head by the row's position
// (cos_sin [max_pos, rd]: rd/2 cos | rd/2 sin, frequency scaling folded in): `half` pairs (i, i + rd/2),
// else (2i, 2i + 1); the other dims pass through.  Everything is computed in fp32.
//
// Cache layout per layer: k [num_blocks, G, block_size, dk], v [num_blocks, G, block_size, dv].
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

constexpr int MAXHEADS = 512;     // q + k heads of a row (their sums of squares sit in LDS)

template <typename T>
__global__ __launch_bounds__(256) void qk_prep_kernel(T* __restrict__ qkv, int stride, const int* __restrict__ positions,
                                                      const int* __restrict__ slots, const float* __restrict__ qw,
                                                      const float* __restrict__ kw, float eps,
                                                      const float* __restrict__ cos_sin, int rd, int H, int G, int dk,
                                                      int dv, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                      int block_size, int full, int half) {
  __shared__ float inv[MAXHEADS];          // 1 / rms of every head (all equal inside q / inside k when `full`)
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  T* row = qkv + (size_t)t * stride;
  const int slot = slots[t];
  const int blk = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? slot - blk * block_size : 0;
  const float* cs = rd > 0 ? cos_sin + (size_t)positions[t] * rd : nullptr;
  const int rh = rd >> 1;

  for (int head = wave; head < H + G; head += 4) {
    const T* hp = row + (size_t)head * dk;
    float ss = 0.f;
    for (int e = lane; e < dk; e += 64) {
      const float x = ldf<T>(hp + e);
      ss += x * x;
    }
    ss = wave_sum(ss);
    if (lane == 0) inv[head] = ss;
  }
  __syncthreads();
  if (full) {
    // wave 0 sums the q heads, wave 1 the k heads
    if (wave < 2) {
      const int h0 = wave == 0 ? 0 : H, nh = wave == 0 ? H : G;
      float ss = 0.f;
      for (int h = lane; h < nh; h += 64) ss += inv[h0 + h];
      ss = wave_sum(ss);
      const float r = 1.f / sqrtf(ss / (float)(nh * dk) + eps);
      __builtin_amdgcn_wave_barrier();
      for (int h = lane; h < nh; h += 64) inv[h0 + h] = r;
    }
  } else {
    for (int h = threadIdx.x; h < H + G; h += 256) inv[h] = 1.f / sqrtf(inv[h] / (float)dk + eps);
  }
  __syncthreads();

  // units: per head, rh rotation pairs and dk - rd pass-through dims
  const int upd = rh + (dk - rd);
  const int total = (H + G) * upd;
  for (int i = threadIdx.x; i < total; i += 256) {
    const int head = i / upd, u = i - head * upd;
    const bool is_k = head >= H;
    if (is_k && slot < 0) continue;
    T* src = row + (size_t)head * dk;
    T* dst = is_k ? k_cache + (((size_t)blk * G + (head - H)) * block_size + off) * dk : src;
    const float* nw = is_k ? kw + (full ? (size_t)(head - H) * dk : 0) : qw + (full ? (size_t)head * dk : 0);
    const float r = inv[head];
    if (u < rh) {
      const int e0 = half ? u : 2 * u, e1 = half ? u + rh : 2 * u + 1;
      const float x = ldf<T>(src + e0) * r * nw[e0], y = ldf<T>(src + e1) * r * nw[e1];
      const float c = cs[u], sn = cs[rh + u];
      stf<T>(dst + e0, x * c - y * sn);
      stf<T>(dst + e1, y * c + x * sn);
    } else {
      const int e = rd + (u - rh);
      stf<T>(dst + e, ldf<T>(src + e) * r * nw[e]);
    }
  }
  if (slot >= 0) {
    const T* vsrc = row + (size_t)(H + G) * dk;
    for (int i = threadIdx.x; i < G * dv; i += 256) {
      const int vh = i / dv, d = i - vh * dv;
      v_cache[(((size_t)blk * G + vh) * block_size + off) * dv + d] = vsrc[i];
    }
  }
}


// 16 bytes of activations as floats (8 bf16 or 4 fp32) and back
template <typename T> struct Chunk;
template <> struct Chunk<uint16_t> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void load(const uint16_t* p, float* f) { unpack8(*reinterpret_cast<const u32x4*>(p), f); }
  static __device__ __forceinline__ void store(uint16_t* p, const float* f) { *reinterpret_cast<u32x4*>(p) = pack8(f); }
};
template <> struct Chunk<float> {
  static constexpr int E = 4;
  static __device__ __forceinline__ void load(const float* p, float* f) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
  }
  static __device__ __forceinline__ void store(float* p, const float* f) {
    *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
  }
};

__device__ __forceinline__ float row16_total(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));
  return v;
}

// The same step in 16-byte chunks: head size, rotated span (its half for the half-split pairing), value size and row
// stride are multiples of a chunk.  Sums of squares: sixteen lanes per head; then one thread per chunk (pair of chunks
// for the half-split pairing) normalises, rotates and stores.
template <typename T>
__global__ __launch_bounds__(256) void qk_prep_vec_kernel(T* __restrict__ qkv, int stride, const int* __restrict__ positions,
                                                          const int* __restrict__ slots, const float* __restrict__ qw,
                                                          const float* __restrict__ kw, float eps,
                                                          const float* __restrict__ cos_sin, int rd, int H, int G, int dk,
                                                          int dv, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                          int block_size, int full, int half) {
  constexpr int E = Chunk<T>::E;
  __shared__ float inv[MAXHEADS];
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * stride;
  const int slot = slots[t];
  const int blk = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? slot - blk * block_size : 0;
  const float* cs = rd > 0 ? cos_sin + (size_t)positions[t] * rd : nullptr;
  const int rh = rd >> 1;
  const int nch = dk / E;
  const int l = threadIdx.x & 15;
  for (int head = threadIdx.x >> 4; head < H + G; head += 16) {
    const T* hp = row + (size_t)head * dk;
    float ss = 0.f;
    for (int c = l; c < nch; c += 16) {
      float x[E];
      Chunk<T>::load(hp + c * E, x);
#pragma unroll
      for (int j = 0; j < E; ++j) ss += x[j] * x[j];
    }
    ss = row16_total(ss);
    if (l == 0) inv[head] = ss;
  }
  __syncthreads();
  if (full) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (wave < 2) {
      const int h0 = wave == 0 ? 0 : H, nh = wave == 0 ? H : G;
      float ss = 0.f;
      for (int h = lane; h < nh; h += 64) ss += inv[h0 + h];
      ss = wave_sum(ss);
      const float r = 1.f / sqrtf(ss / (float)(nh * dk) + eps);
      __builtin_amdgcn_wave_barrier();
      for (int h = lane; h < nh; h += 64) inv[h0 + h] = r;
    }
  } else {
    for (int h = threadIdx.x; h < H + G; h += 256) inv[h] = 1.f / sqrtf(inv[h] / (float)dk + eps);
  }
  __syncthreads();

  // units per head: half-split pairing: rh / E chunk pairs + (dk - rd) / E plain chunks; interleaved: dk / E chunks
  const int npair = half ? rh / E : 0;
  const int upd = half ? npair + (dk - rd) / E : nch;
  const int total = (H + G) * upd;
  for (int i = threadIdx.x; i < total; i += 256) {
    const int head = i / upd, u = i - head * upd;
    const bool is_k = head >= H;
    if (is_k && slot < 0) continue;
    T* src = row + (size_t)head * dk;
    T* dst = is_k ? k_cache + (((size_t)blk * G + (head - H)) * block_size + off) * dk : src;
    const float* nw = is_k ? kw + (full ? (size_t)(head - H) * dk : 0) : qw + (full ? (size_t)head * dk : 0);
    const float r = inv[head];
    if (half && u < npair) {
      const int e0 = u * E, e1 = e0 + rh;
      float x[E], y[E], o0[E], o1[E];
      Chunk<T>::load(src + e0, x);
      Chunk<T>::load(src + e1, y);
#pragma unroll
      for (int j = 0; j < E; ++j) {
        const float a = x[j] * r * nw[e0 + j], b = y[j] * r * nw[e1 + j];
        const float c = cs[e0 + j], sn = cs[rh + e0 + j];
        o0[j] = a * c - b * sn;
        o1[j] = b * c + a * sn;
      }
      Chunk<T>::store(dst + e0, o0);
      Chunk<T>::store(dst + e1, o1);
    } else {
      const int e0 = half ? rd + (u - npair) * E : u * E;
      float x[E], o[E];
      Chunk<T>::load(src + e0, x);
#pragma unroll
      for (int j = 0; j < E; ++j) o[j] = x[j] * r * nw[e0 + j];
      if (!half && e0 < rd) {                      // interleaved pairs (2i, 2i + 1) inside the chunk (rd a multiple of E)
#pragma unroll
        for (int j = 0; j < E; j += 2) {
          const float c = cs[(e0 + j) >> 1], sn = cs[rh + ((e0 + j) >> 1)];
          const float a = o[j], b = o[j + 1];
          o[j] = a * c - b * sn;
          o[j + 1] = b * c + a * sn;
        }
      }
      Chunk<T>::store(dst + e0, o);
    }
  }
  if (slot >= 0) {
    const T* vsrc = row + (size_t)(H + G) * dk;
    const int cpv = dv / E;
    for (int i = threadIdx.x; i < G * cpv; i += 256) {
      const int vh = i / cpv, c = i - vh * cpv;
      *reinterpret_cast<u32x4*>(v_cache + (((size_t)blk * G + vh) * block_size + off) * dv + c * E) =
          *reinterpret_cast<const u32x4*>(vsrc + (size_t)vh * dv + c * E);
    }
  }
}

}  // namespace

extern "C" int dgi_qk_prep(void* qkv, int is_f32, int T, int stride, const int* positions, const int* slots,
                           const float* qw, const float* kw, float eps, const float* cos_sin, int rd, int H, int G,
                           int dk, int dv, void* k_cache, void* v_cache, int block_size, int full, int half,
                           hipStream_t s) {
  if (T == 0) return 0;
  if (rd < 0 || rd > dk || (rd & 1) || (rd > 0 && !cos_sin)) return -2;
  if (H + G > MAXHEADS || H <= 0 || G <= 0) return -3;
  {
    const int E = is_f32 ? 4 : 8;
    const bool vec = dk % E == 0 && dv % E == 0 && stride % E == 0 && rd % E == 0 && (!half || (rd / 2) % E == 0) &&
                     (((uintptr_t)qkv | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0;
    if (vec) {
      if (is_f32)
        qk_prep_vec_kernel<float><<<T, 256, 0, s>>>((float*)qkv, stride, positions, slots, qw, kw, eps, cos_sin, rd, H, G, dk,
                                                    dv, (float*)k_cache, (float*)v_cache, block_size, full, half);
      else
        qk_prep_vec_kernel<uint16_t><<<T, 256, 0, s>>>((uint16_t*)qkv, stride, positions, slots, qw, kw, eps, cos_sin, rd, H,
                                                       G, dk, dv, (uint16_t*)k_cache, (uint16_t*)v_cache, block_size, full,
                                                       half);
      DGI_CHECK_LAUNCH();
      return 0;
    }
  }
  if (is_f32)
    qk_prep_kernel<float><<<T, 256, 0, s>>>((float*)qkv, stride, positions, slots, qw, kw, eps, cos_sin, rd, H, G, dk, dv,
                                            (float*)k_cache, (float*)v_cache, block_size, full, half);
  else
    qk_prep_kernel<uint16_t><<<T, 256, 0, s>>>((uint16_t*)qkv, stride, positions, slots, qw, kw, eps, cos_sin, rd, H, G,
                                               dk, dv, (uint16_t*)k_cache, (uint16_t*)v_cache, block_size, full, half);
  DGI_CHECK_LAUNCH();
  return 0;
}
