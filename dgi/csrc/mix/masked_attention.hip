// dgi/csrc/mix/masked_attention.hip — row-wise softmax attention over the paged KV pool for any
// head geometry, in bf16 or fp32, with a block ("chunk") mask and an output gate.
//
// decode_attention.hip and prefill_attention.hip are MFMA kernels for bf16 heads of 64 / 128
// dims whose keys and values share one size.  This kernel is the general form the other
// geometries run on (key size != value size, sizes that are no multiple of 16, fp32 caches)
// and the one both step phases share: every query row — a decode row or one row of a prompt
// portion — is one wave that walks its own visible keys
//
//     [first(p), p],   first(p) = floor(p / mask) * mask   (mask > 0: keys of the row's own block
//                                                            of `mask` positions, counted from
//                                                            position 0 of the sequence)
//                      first(p) = 0                          (mask == 0: plain causal)
//
// straight from the cache (this step's keys are written before it runs), so the result does
// not depend on how the prompt was cut into steps or on what else is in the batch.
// Scores, the online softmax and the output accumulation are fp32; exp is the accurate expf.
// Optional distance bias: dist_bias[min(p - j, n_dist - 1)][head] (fp32, one row per distance, the
// last row for everything farther) is added to the scaled score of key j before the softmax.
// Optional soft cap: the scaled (and biased) score s becomes softcap * tanh(s / softcap).
// Optional sinks: exp(sinks[head]) joins the softmax denominator of that head (a logit that has no
// key and no value; it is neither scaled nor capped).
// Optional epilogue: out *= sigmoid(gate) element by element (the mixer's output gate, read
// from the same fused projection row as q).
//
// Wave layout: lane j scores key first + 64 i + j (a contiguous dk-vector per lane, 16-byte
// loads where dk allows); the 64 probabilities go through LDS and every lane accumulates the
// value dims d = lane + 64 c, so the V reads of one key are one coalesced row.
// grid = (rows, H), 64 threads.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

constexpr int MAXC = 8;       // value dims per lane: dv <= 64 * MAXC
constexpr int MAXDK = 512;    // query vector staged in LDS

__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const float* __restrict__ k, int dk) {
  float acc = 0.f;
  if ((dk & 3) == 0) {
    for (int e = 0; e < dk; e += 4) {
      const float4 v = *reinterpret_cast<const float4*>(k + e);
      acc += qs[e] * v.x + qs[e + 1] * v.y + qs[e + 2] * v.z + qs[e + 3] * v.w;
    }
  } else {
    for (int e = 0; e < dk; ++e) acc += qs[e] * k[e];
  }
  return acc;
}

__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const uint16_t* __restrict__ k, int dk) {
  float acc = 0.f;
  if ((dk & 7) == 0) {
    for (int e = 0; e < dk; e += 8) {
      float f[8];
      unpack8(*reinterpret_cast<const u32x4*>(k + e), f);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += qs[e + j] * f[j];
    }
  } else {
    for (int e = 0; e < dk; ++e) acc += qs[e] * bf16_to_f32(k[e]);
  }
  return acc;
}

template <typename T>
__global__ __launch_bounds__(64) void masked_attn_rows_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ cu_seqlens, int n_seqs,
    const int* __restrict__ positions, int G, int dk, int dv, int bs, float scale, int mask,
    const T* __restrict__ gate, int gate_stride, T* __restrict__ out, int out_stride,
    const float* __restrict__ dist_bias, int n_dist, float softcap, const float* __restrict__ sinks) {
  __shared__ float qs[MAXDK];
  __shared__ float ps[64];
  __shared__ long long vo[64];

  const int row = blockIdx.x, head = blockIdx.y, H = gridDim.y;
  const int lane = threadIdx.x;
  const int kvh = head / (H / G);
  // the row's sequence: row index itself (decode rows), or the portion holding it (cu_seqlens)
  int seq = row;
  if (cu_seqlens) {
    int lo = 0, hi = n_seqs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_seqlens[mid] <= row) lo = mid; else hi = mid - 1;
    }
    seq = lo;
  }
  const int* bt = block_tables + (size_t)seq * bt_stride;
  const int pos = positions[row];
  const int first = mask > 0 ? (pos / mask) * mask : 0;

  const T* qp = q + (size_t)row * q_stride + (size_t)head * dk;
  for (int e = lane; e < dk; e += 64) qs[e] = ldf<T>(qp + e);
  __syncthreads();

  float m_run = -__builtin_inff(), l_run = 0.f;
  float o[MAXC];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) o[c] = 0.f;
  const int nc = (dv + 63) >> 6;

  for (int k0 = first; k0 <= pos; k0 += 64) {
    const int key = k0 + lane;
    const bool ok = key <= pos;
    float s = -__builtin_inff();
    long long vbase = 0;
    if (ok) {
      const int blk = bt[key / bs];
      const long long slot = ((long long)blk * G + kvh) * bs + (key % bs);
      s = dot_row(qs, k_cache + slot * dk, dk) * scale;
      if (dist_bias) s += dist_bias[(size_t)min(pos - key, n_dist - 1) * H + head];
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      vbase = slot * dv;
    }
    const float m_new = fmaxf(m_run, wave_max(s));     // lane 0's key k0 is always visible: finite
    const float p = ok ? expf(s - m_new) : 0.f;
    const float corr = expf(m_run - m_new);            // first tile: exp(-inf) = 0
    l_run = l_run * corr + wave_sum(p);
    m_run = m_new;
    __syncthreads();                                   // previous tile's ps / vo fully read
    ps[lane] = p;
    vo[lane] = vbase;
    __syncthreads();
    const int n = min(64, pos - k0 + 1);
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nc) {
        const int d = lane + 64 * c;
        float acc = o[c] * corr;
        if (d < dv)
          for (int j = 0; j < n; ++j) acc += ps[j] * ldf<T>(v_cache + vo[j] + d);
        o[c] = acc;
      }
    }
  }
  float inv = 1.f / l_run;
  if (sinks) {
    // the sink logit joins the denominator only: out = o / (l + exp(sink - m)), with the larger of the two as reference
    const float sk = sinks[head], m2 = fmaxf(m_run, sk);
    const float f = expf(m_run - m2);
    inv = f / (l_run * f + expf(sk - m2));
  }
  T* op = out + (size_t)row * out_stride + (size_t)head * dv;
  const T* gp = gate ? gate + (size_t)row * gate_stride + (size_t)head * dv : nullptr;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int d = lane + 64 * c;
    if (c < nc && d < dv) {
      float v = o[c] * inv;
      if (gp) v *= 1.f / (1.f + expf(-ldf<T>(gp + d)));
      stf<T>(op + d, v);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Grouped kernel: one workgroup per (row, kv head) serves all R = H / G query heads of the group
// from ONE pass over the keys, with 16-byte cache reads.  Eight waves take 64-key tiles round
// robin; in a tile lane j scores key j against the R staged queries (its K row is read once),
// the probabilities go through LDS, and for the values a 16-lane group owns one key at a time
// (lane c of the group its 16-byte chunk c), so one wave instruction reads four whole V rows.
// Partial outputs are combined over the four lane groups by shuffles and over the waves in LDS.
// Needs dk, dv multiples of 8 (bf16) / 4 (fp32), H / G <= 8 and (H / G) * dv <= 1024.
constexpr int GNW = 8;        // waves per workgroup

template <typename T, int R, int VP>
__global__ __launch_bounds__(64 * GNW) void masked_attn_group_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ cu_seqlens, int n_seqs,
    const int* __restrict__ positions, int H, int dk, int dv, int bs, float scale, int mask,
    const T* __restrict__ gate, int gate_stride, T* __restrict__ out, int out_stride,
    const float* __restrict__ dist_bias, int n_dist, float softcap, const float* __restrict__ sinks) {
  constexpr int E = 16 / sizeof(T);
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int row = blockIdx.x, kvh = blockIdx.y, G = gridDim.y;
  const int r = H / G;
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63;
  const int lg = lane >> 4, lc = lane & 15;
  float* qs = smem;                                  // [R][dk]
  float* ps = qs + R * dk;                           // [GNW][R][64]
  int* vs = reinterpret_cast<int*>(ps + GNW * R * 64);   // [GNW][64] cache slot of each key of the wave's tile
  float* cm = reinterpret_cast<float*>(vs + GNW * 64);   // [GNW][R] running max, then [GNW][R] sums
  float* co = cm + 2 * GNW * R;                      // [GNW][R][dv] partial outputs

  int seq = row;
  if (cu_seqlens) {
    int lo = 0, hi = n_seqs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_seqlens[mid] <= row) lo = mid; else hi = mid - 1;
    }
    seq = lo;
  }
  const int* bt = block_tables + (size_t)seq * bt_stride;
  const int pos = positions[row];
  const int first = mask > 0 ? (pos / mask) * mask : 0;

  const T* qp = q + (size_t)row * q_stride + (size_t)kvh * r * dk;
  for (int e = tid; e < r * dk; e += 64 * GNW) qs[e] = ldf<T>(qp + e);
  __syncthreads();

  float m[R], l[R], o[R][VP][E];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    m[i] = -__builtin_inff();
    l[i] = 0.f;
#pragma unroll
    for (int p = 0; p < VP; ++p)
#pragma unroll
      for (int j = 0; j < E; ++j) o[i][p][j] = 0.f;
  }
  float* psw = ps + w * R * 64;
  int* vsw = vs + w * 64;
  const int ntiles = (pos - first) / 64 + 1;
  for (int tile = w; tile < ntiles; tile += GNW) {
    const int k0 = first + tile * 64;
    const int key = k0 + lane;
    const bool ok = key <= pos;
    float sc[R];
#pragma unroll
    for (int i = 0; i < R; ++i) sc[i] = 0.f;
    int slot = 0;
    if (ok) {
      slot = (bt[key / bs] * G + kvh) * bs + (key % bs);
      const T* kp = k_cache + (size_t)slot * dk;
      for (int e = 0; e < dk; e += E) {
        float kf[E];
        const u32x4 kv = *reinterpret_cast<const u32x4*>(kp + e);
        if constexpr (sizeof(T) == 2) {
          unpack8(kv, kf);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) kf[j] = __uint_as_float(kv[j]);
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
          if (i < r) {
            const float* qi = qs + i * dk + e;
#pragma unroll
            for (int j = 0; j < E; ++j) sc[i] += qi[j] * kf[j];
          }
        }
      }
    }
    // this wave's previous tile is fully consumed (its LDS reads were issued, in order, before)
#pragma unroll
    for (int i = 0; i < R; ++i) {
      if (i < r) {
        float s = -__builtin_inff();
        if (ok) {
          s = sc[i] * scale;
          if (dist_bias) s += dist_bias[(size_t)min(pos - key, n_dist - 1) * H + kvh * r + i];
          if (softcap > 0.f) s = softcap * tanhf(s / softcap);
        }
        const float m_new = fmaxf(m[i], wave_max(s));       // key k0 (lane 0) is visible: finite
        const float p = ok ? expf(s - m_new) : 0.f;
        const float corr = expf(m[i] - m_new);
        l[i] = l[i] * corr + wave_sum(p);
        m[i] = m_new;
#pragma unroll
        for (int vp = 0; vp < VP; ++vp)
#pragma unroll
          for (int j = 0; j < E; ++j) o[i][vp][j] *= corr;
        psw[i * 64 + lane] = p;
      }
    }
    vsw[lane] = slot;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int n = min(64, pos - k0 + 1);
    for (int kk = lg; kk < n; kk += 4) {
      const T* vp_ = v_cache + (size_t)vsw[kk] * dv;
      float pk[R];
#pragma unroll
      for (int i = 0; i < R; ++i) pk[i] = i < r ? psw[i * 64 + kk] : 0.f;
#pragma unroll
      for (int vp = 0; vp < VP; ++vp) {
        const int c = (lc + 16 * vp) * E;
        if (c < dv) {
          float vf[E];
          const u32x4 vv = *reinterpret_cast<const u32x4*>(vp_ + c);
          if constexpr (sizeof(T) == 2) {
            unpack8(vv, vf);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) vf[j] = __uint_as_float(vv[j]);
          }
#pragma unroll
          for (int i = 0; i < R; ++i)
#pragma unroll
            for (int j = 0; j < E; ++j) o[i][vp][j] += pk[i] * vf[j];
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  // lane groups -> lane group 0, then waves -> LDS
#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int vp = 0; vp < VP; ++vp)
#pragma unroll
      for (int j = 0; j < E; ++j) {
        float v = o[i][vp][j];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        o[i][vp][j] = v;
      }
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      cm[w * R + i] = m[i];
      cm[GNW * R + w * R + i] = l[i];
    }
  }
  if (lg == 0) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (i < r)
#pragma unroll
        for (int vp = 0; vp < VP; ++vp) {
          const int c = (lc + 16 * vp) * E;
          if (c < dv)
#pragma unroll
            for (int j = 0; j < E; ++j) co[((size_t)w * R + i) * dv + c + j] = o[i][vp][j];
        }
  }
  __syncthreads();
  for (int idx = tid; idx < r * dv; idx += 64 * GNW) {
    const int i = idx / dv, d = idx - i * dv;
    const int head = kvh * r + i;
    float M = sinks ? sinks[head] : -__builtin_inff();
#pragma unroll
    for (int ww = 0; ww < GNW; ++ww) M = fmaxf(M, cm[ww * R + i]);
    float L = sinks ? expf(sinks[head] - M) : 0.f, O = 0.f;      // the sink: one more term of the denominator
#pragma unroll
    for (int ww = 0; ww < GNW; ++ww) {
      const float f = expf(cm[ww * R + i] - M);          // waves without a tile: exp(-inf) = 0
      L += cm[GNW * R + ww * R + i] * f;
      O += co[((size_t)ww * R + i) * dv + d] * f;
    }
    float v = O / L;
    if (gate) v *= 1.f / (1.f + expf(-ldf<T>(gate + (size_t)row * gate_stride + (size_t)head * dv + d)));
    stf<T>(out + (size_t)row * out_stride + (size_t)head * dv + d, v);
  }
}

template <typename T, int R, int VP>
int launch_group(const void* q, int q_stride, const void* k_cache, const void* v_cache, const int* block_tables,
                 int bt_stride, const int* cu_seqlens, int n_seqs, const int* positions, int rows, int H, int G, int dk,
                 int dv, int bs, float scale, int mask, const void* gate, int gate_stride, void* out, int out_stride,
                 const float* dist_bias, int n_dist, float softcap, const float* sinks, hipStream_t s) {
  const size_t lds = (size_t)(R * dk + GNW * R * 64 + GNW * 64 + 2 * GNW * R + GNW * R * dv) * 4;
  if (lds > 64 * 1024) return -1;
  masked_attn_group_kernel<T, R, VP><<<dim3(rows, G), 64 * GNW, lds, s>>>(
      (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, block_tables, bt_stride, cu_seqlens, n_seqs,
      positions, H, dk, dv, bs, scale, mask, (const T*)gate, gate_stride, (T*)out, out_stride, dist_bias, n_dist,
      softcap, sinks);
  return 0;
}

template <typename T>
int dispatch_group(int r, int vpn, const void* q, int q_stride, const void* k_cache, const void* v_cache,
                   const int* block_tables, int bt_stride, const int* cu_seqlens, int n_seqs, const int* positions,
                   int rows, int H, int G, int dk, int dv, int bs, float scale, int mask, const void* gate,
                   int gate_stride, void* out, int out_stride, const float* dist_bias, int n_dist, float softcap,
                   const float* sinks, hipStream_t s) {
#define DGI_GRP(RV, VPV)                                                                                       \
  return launch_group<T, RV, VPV>(q, q_stride, k_cache, v_cache, block_tables, bt_stride, cu_seqlens, n_seqs, \
                                  positions, rows, H, G, dk, dv, bs, scale, mask, gate, gate_stride, out, out_stride, dist_bias, \
                                  n_dist, softcap, sinks, s)
  if (vpn == 1) {
    if (r == 1) DGI_GRP(1, 1);
    if (r == 2) DGI_GRP(2, 1);
    if (r <= 4) DGI_GRP(4, 1);
    DGI_GRP(8, 1);
  }
  if (r == 1) DGI_GRP(1, 2);
  if (r == 2) DGI_GRP(2, 2);
  if (r <= 4) DGI_GRP(4, 2);
  DGI_GRP(8, 2);
#undef DGI_GRP
}

}  // namespace

// q / gate / out: row-major with their own row strides (elements); cu_seqlens (n_seqs + 1 row
// offsets) maps rows to block-table rows, nullptr: row i uses block-table row i.
extern "C" int dgi_masked_attn_rows(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                    const int* block_tables, int bt_stride, const int* cu_seqlens, int n_seqs,
                                    const int* positions, int rows, int H, int G, int dk, int dv, int block_size,
                                    float scale, int mask, const void* gate, int gate_stride, void* out,
                                    int out_stride, int is_f32, const float* dist_bias, int n_dist, float softcap,
                                    const float* sinks, hipStream_t s) {
  if (rows == 0) return 0;
  if (G <= 0 || H % G) return -2;
  if (dk > MAXDK || dv > 64 * MAXC || dk <= 0 || dv <= 0) return -3;
  if (H > 65535 || mask < 0) return -4;
  if (dist_bias && n_dist < 1) return -5;
  {
    // grouped kernel where the geometry allows (see masked_attn_group_kernel)
    const int E = is_f32 ? 4 : 8, r = H / G;
    const int vpn = (dv + 16 * E - 1) / (16 * E);
    const bool aligned = ((uintptr_t)k_cache | (uintptr_t)v_cache) % 16 == 0;
    if (dk % E == 0 && dv % E == 0 && r <= 8 && vpn <= 2 && r * dv <= 1024 && aligned && G <= 65535) {
      const int rc = is_f32 ? dispatch_group<float>(r, vpn, q, q_stride, k_cache, v_cache, block_tables, bt_stride, cu_seqlens,
                                                    n_seqs, positions, rows, H, G, dk, dv, block_size, scale, mask, gate,
                                                    gate_stride, out, out_stride, dist_bias, n_dist, softcap, sinks, s)
                            : dispatch_group<uint16_t>(r, vpn, q, q_stride, k_cache, v_cache, block_tables, bt_stride,
                                                       cu_seqlens, n_seqs, positions, rows, H, G, dk, dv, block_size, scale,
                                                       mask, gate, gate_stride, out, out_stride, dist_bias, n_dist, softcap,
                                                       sinks, s);
      if (rc == 0) {
        DGI_CHECK_LAUNCH();
        return 0;
      }
    }
  }
  const dim3 grid(rows, H);
  if (is_f32)
    masked_attn_rows_kernel<float><<<grid, 64, 0, s>>>(
        (const float*)q, q_stride, (const float*)k_cache, (const float*)v_cache, block_tables, bt_stride, cu_seqlens,
        n_seqs, positions, G, dk, dv, block_size, scale, mask, (const float*)gate, gate_stride, (float*)out, out_stride,
        dist_bias, n_dist, softcap, sinks);
  else
    masked_attn_rows_kernel<uint16_t><<<grid, 64, 0, s>>>(
        (const uint16_t*)q, q_stride, (const uint16_t*)k_cache, (const uint16_t*)v_cache, block_tables, bt_stride,
        cu_seqlens, n_seqs, positions, G, dk, dv, block_size, scale, mask, (const uint16_t*)gate, gate_stride,
        (uint16_t*)out, out_stride, dist_bias, n_dist, softcap, sinks);
  DGI_CHECK_LAUNCH();
  return 0;
}
