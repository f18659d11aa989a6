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

}  // namespace

extern "C" int dgi_qk_prep(void* qkv, int is_f32, int T, int stride, const int* positions, const int* slots,
                           const float* qw, const float* kw, float eps, const float* cos_sin, int rd, int H, int G,
                           int dk, int dv, void* k_cache, void* v_cache, int block_size, int full, int half,
                           hipStream_t s) {
  if (T == 0) return 0;
  if (rd < 0 || rd > dk || (rd & 1) || (rd > 0 && !cos_sin)) return -2;
  if (H + G > MAXHEADS || H <= 0 || G <= 0) return -3;
  if (is_f32)
    qk_prep_kernel<float><<<T, 256, 0, s>>>((float*)qkv, stride, positions, slots, qw, kw, eps, cos_sin, rd, H, G, dk, dv,
                                            (float*)k_cache, (float*)v_cache, block_size, full, half);
  else
    qk_prep_kernel<uint16_t><<<T, 256, 0, s>>>((uint16_t*)qkv, stride, positions, slots, qw, kw, eps, cos_sin, rd, H, G,
                                               dk, dv, (uint16_t*)k_cache, (uint16_t*)v_cache, block_size, full, half);
  DGI_CHECK_LAUNCH();
  return 0;
}
