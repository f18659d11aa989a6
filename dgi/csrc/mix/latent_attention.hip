// dgi/csrc/mix/latent_attention.hip — softmax attention over cached latents, for decode rows and
// prompt rows alike, in bf16 or fp32.
//
// The cache holds ONE row per token, [c | r]: the normalised key/value latent c (kr dims) and a
// rotated key part r (rd dims) that all heads share.  With the unrotated query part folded through
// the key up-projection beforehand (q_lat [H, T, kr]) head h's score of key j is
//
//     s = (q_lat[h] . c_j + rot(q_rot[h]) . r_j) * scale
//
// and its output the probability-weighted sum of the c_j (the value up-projection follows as a
// batched GEMM).  So every head reads the same cached row, as key and as value.  A workgroup
// therefore owns one query row and a group of heads, one wave per head: tiles of KT cached rows
// are staged in LDS once (16-byte copies, rows padded against bank conflicts) and every wave
// scores them (lane j: key j of the tile) and accumulates its weighted sum from LDS (lane l: E
// consecutive latent dims, one 16-byte LDS read per key).  The row's visible keys are
//
//     [max(0, p - window + 1), p]   (window > 0: the last `window` positions, itself included)
//     [0, p]                        (window == 0)
//
// read straight from the pages (this step's rows are written before the kernel runs), so the
// result does not depend on how a prompt was cut into steps or on what else is in the batch.
// The query's rotated part is rotated here, while it is staged (interleaved pairs or halves).
// Scores, the online softmax and the accumulation are fp32; exp is the accurate expf.
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

// E elements (16 bytes) as floats
template <typename T> __device__ __forceinline__ void ld16(const T* p, float* f);
template <> __device__ __forceinline__ void ld16<uint16_t>(const uint16_t* p, float* f) {
  unpack8(*reinterpret_cast<const u32x4*>(p), f);
}
template <> __device__ __forceinline__ void ld16<float>(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}

// VEC: 16-byte accesses (kr and kr + rd multiples of E = 16 / sizeof(T), aligned cache); else element-wise.
// KT keys per tile (<= 64).  Value chunks per lane: VEC: kr <= 64 * E * MAXC; scalar: kr <= 64 * MAXC.
template <typename T, bool VEC, int KT>
__global__ __launch_bounds__(1024) void latent_attn_rows_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ q_lat, long long ql_hs, long long ql_ts,
    const T* __restrict__ cache, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_seqlens, int n_seqs, const int* __restrict__ positions, int H, int dim, int rd, int kr,
    int bs, float scale, int window, const float* __restrict__ cos_sin, int dims, int interleaved, T* __restrict__ out,
    long long o_hs, long long o_ts, int DP, int DQ, float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int E = 16 / sizeof(T);
  constexpr int CE = VEC ? E : 1;                    // elements per value chunk
  constexpr int MAXC = VEC ? (sizeof(T) == 2 ? 2 : 4) : 8;
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int nw = blockDim.x >> 6;
  const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
  T* tile = reinterpret_cast<T*>(smem);                                  // [KT][DP]
  float* qs = smem + ((size_t)KT * DP * sizeof(T) + 3) / 4;               // [nw][DQ]
  float* ps = qs + (size_t)nw * DQ;                                       // [nw][KT]
  const int D = kr + rd;
  const int row = blockIdx.x;
  const int head_raw = blockIdx.y * nw + w;
  const int head = min(head_raw, H - 1);            // a spare wave shadows the last head and stores nothing

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
  const int first = window > 0 ? max(0, pos - window + 1) : 0;

  // this wave's query: folded part, then the rotated part
  float* qw = qs + (size_t)w * DQ;
  {
    const T* ql = q_lat + (size_t)head * ql_hs + (size_t)row * ql_ts;
    for (int e = lane; e < kr; e += 64) qw[e] = ldf<T>(ql + e);
    const T* qr = q + (size_t)row * q_stride + (size_t)head * (dim + rd) + dim;
    const int half = dims >> 1;
    const float* cs = cos_sin ? cos_sin + (size_t)pos * dims : nullptr;
    for (int i = lane; i < half; i += 64) {
      const int i0 = interleaved ? 2 * i : i, i1 = interleaved ? 2 * i + 1 : i + half;
      const float u = ldf<T>(qr + i0), v = ldf<T>(qr + i1);
      const float c = cs[i], s = cs[half + i];
      qw[kr + i0] = u * c - v * s;
      qw[kr + i1] = v * c + u * s;
    }
    for (int e = dims + lane; e < rd; e += 64) qw[kr + e] = ldf<T>(qr + e);
  }

  float m_run = -__builtin_inff(), l_run = 0.f;
  float o[MAXC][CE];
#pragma unroll
  for (int c = 0; c < MAXC; ++c)
#pragma unroll
    for (int j = 0; j < CE; ++j) o[c][j] = 0.f;
  const int nchunk = (kr + CE - 1) / CE;            // value chunks of the latent

  // the row's key tiles, cut into gridDim.z contiguous runs (one workgroup each; a run may be empty)
  const int ntiles = (pos - first + KT) / KT;
  const int tps = (ntiles + (int)gridDim.z - 1) / (int)gridDim.z;
  const int t_hi = min(ntiles, ((int)blockIdx.z + 1) * tps);
  for (int ti = blockIdx.z * tps; ti < t_hi; ++ti) {
    const int k0 = first + ti * KT;
    const int n = min(KT, pos - k0 + 1);
    __syncthreads();                                 // the previous tile is fully read (and qs written)
    if constexpr (VEC) {
      const int cpr = D / E;
      for (int i = threadIdx.x; i < n * cpr; i += blockDim.x) {
        const int j = i / cpr, c = i - j * cpr;
        const int key = k0 + j;
        const long long slot = (long long)bt[key / bs] * bs + (key % bs);
        *reinterpret_cast<u32x4*>(tile + (size_t)j * DP + c * E) =
            *reinterpret_cast<const u32x4*>(cache + slot * D + c * E);
      }
    } else {
      for (int i = threadIdx.x; i < n * D; i += blockDim.x) {
        const int j = i / D, c = i - j * D;
        const int key = k0 + j;
        const long long slot = (long long)bt[key / bs] * bs + (key % bs);
        tile[(size_t)j * DP + c] = cache[slot * D + c];
      }
    }
    __syncthreads();
    float s = -__builtin_inff();
    const bool ok = lane < n;
    if (ok) {
      const T* kp = tile + (size_t)lane * DP;
      float acc = 0.f;
      if constexpr (VEC) {
        for (int e = 0; e < D; e += E) {
          float f[E];
          ld16<T>(kp + e, f);
#pragma unroll
          for (int j = 0; j < E; ++j) acc += qw[e + j] * f[j];
        }
      } else {
        for (int e = 0; e < D; ++e) acc += qw[e] * ldf<T>(kp + e);
      }
      s = acc * scale;
    }
    const float m_new = fmaxf(m_run, wave_max(s));     // lane 0's key k0 is always visible: finite
    const float p = ok ? expf(s - m_new) : 0.f;
    const float corr = expf(m_run - m_new);            // first tile: exp(-inf) = 0
    l_run = l_run * corr + wave_sum(p);
    m_run = m_new;
    float* pw = ps + (size_t)w * KT;
    if (lane < KT) pw[lane] = p;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // this wave's ps writes precede its reads below
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int ci = lane + 64 * c;
      if (ci < nchunk) {
        float acc[CE];
#pragma unroll
        for (int j = 0; j < CE; ++j) acc[j] = o[c][j] * corr;
        const T* vp = tile + (size_t)ci * CE;
        for (int j = 0; j < n; ++j) {
          const float pj = pw[j];
          if constexpr (VEC) {
            float f[E];
            ld16<T>(vp + (size_t)j * DP, f);
#pragma unroll
            for (int e = 0; e < E; ++e) acc[e] += pj * f[e];
          } else {
            acc[0] += pj * ldf<T>(vp + (size_t)j * DP);
          }
        }
#pragma unroll
        for (int j = 0; j < CE; ++j) o[c][j] = acc[j];
      }
    }
  }
  if (head_raw >= H) return;
  if (part_o) {
    // one of several runs: unnormalised sums and (max, sum of weights) for latent_attn_reduce_kernel
    const size_t slot = ((size_t)blockIdx.z * H + head) * gridDim.x + row;
    float* po = part_o + slot * kr;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int ci = lane + 64 * c;
      if (ci < nchunk) {
#pragma unroll
        for (int j = 0; j < CE; ++j) po[(size_t)ci * CE + j] = o[c][j];
      }
    }
    if (lane == 0) {
      part_ml[2 * slot] = m_run;
      part_ml[2 * slot + 1] = l_run;
    }
    return;
  }
  const float inv = 1.f / l_run;
  T* op = out + (size_t)head * o_hs + (size_t)row * o_ts;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ci = lane + 64 * c;
    if (ci < nchunk) {
#pragma unroll
      for (int j = 0; j < CE; ++j) stf<T>(op + (size_t)ci * CE + j, o[c][j] * inv);
    }
  }
}

// out[h][row] = sum_z o_z e^(m_z - M) / sum_z l_z e^(m_z - M), M = max_z m_z; grid (rows, H), run 0 is never empty
template <typename T>
__global__ __launch_bounds__(256) void latent_attn_reduce_kernel(const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml, int nsplit, int kr,
                                                                 T* __restrict__ out, long long o_hs, long long o_ts) {
  const int row = blockIdx.x, head = blockIdx.y, rows = gridDim.x, H = gridDim.y;
  float M = -__builtin_inff();
  for (int z = 0; z < nsplit; ++z) M = fmaxf(M, part_ml[2 * (((size_t)z * H + head) * rows + row)]);
  float L = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const size_t slot = ((size_t)z * H + head) * rows + row;
    L += part_ml[2 * slot + 1] * expf(part_ml[2 * slot] - M);
  }
  const float inv = 1.f / L;
  T* op = out + (size_t)head * o_hs + (size_t)row * o_ts;
  for (int e = threadIdx.x; e < kr; e += blockDim.x) {
    float acc = 0.f;
    for (int z = 0; z < nsplit; ++z) {
      const size_t slot = ((size_t)z * H + head) * rows + row;
      acc += part_o[slot * kr + e] * expf(part_ml[2 * slot] - M);
    }
    stf<T>(op + e, acc * inv);
  }
}


// ---------------------------------------------------------------------------------------------
// MFMA form (bf16; kr and kr + rd multiples of 16).  A workgroup owns one query row, a group of 16
// heads and one run of the row's 64-key tiles; its four waves take 16 keys of every tile each and keep
// their own running softmax, so nothing is exchanged between waves per tile.  Per tile and wave:
//
//   S^T [16 keys x 16 heads] = K [16 keys x D] Q^T [D x 16 heads]      D / 16 MFMAs 16x16x16; K rows from LDS;
//                                                                     Q rows stay in LDS beside the tile
//   O^T [kr x 16 heads]     += C^T [kr x 16 keys] P^T [16 keys x 16 heads]    kr / 16 MFMAs
//
// S^T comes out with a lane holding four consecutive keys of one head, which is exactly the operand
// layout P^T needs, and O^T keeps a head's values in the lanes that hold its running maximum, so the
// rescale needs no exchange either.  At the end the four waves' (max, sum, O^T) are combined in LDS and
// the workgroup writes the row's result, or, when the row's keys are cut into gridDim.z runs, one
// partial (max, sum, unnormalised O) per run for latent_attn_reduce_kernel.
template <int NM, int NDS>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(
    const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ q_lat, long long ql_hs, long long ql_ts,
    const uint16_t* __restrict__ cache, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_seqlens, int n_seqs, const int* __restrict__ positions, int H, int dim, int rd, int kr,
    int bs, float scale, int window, const float* __restrict__ cos_sin, int dims, int interleaved, int DP,
    uint16_t* __restrict__ out, long long o_hs, long long o_ts, float* __restrict__ part_o, float* __restrict__ part_ml,
    unsigned cpr_magic) {
  constexpr int KT = 64;
  extern __shared__ __attribute__((aligned(16))) uint16_t qs[];         // [16][DP] the group's queries, then the tile
  uint16_t* tile = qs + (size_t)16 * DP;                                 // [KT][DP]
  const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lr = lane & 15, lg = lane >> 4;
  const int D = kr + rd, nd = D >> 4, nm = kr >> 4;
  const int row = blockIdx.x, rows = gridDim.x, g = blockIdx.y;

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
  const int first = window > 0 ? max(0, pos - window + 1) : 0;

  // the group's queries as bf16 rows [folded part | rotated part]; heads past H are zero rows
  {
    const int half = dims >> 1;
    const float* cs = cos_sin ? cos_sin + (size_t)pos * dims : nullptr;
    // folded part: 16-byte copies where the query tensor allows them (all issued before any lands)
    const bool qvec = ((uintptr_t)q_lat & 15) == 0 && (ql_hs & 7) == 0 && (ql_ts & 7) == 0;
    if (qvec) {
      constexpr int NQ = (16 * NM * 2 + 255) / 256;
      const int cq = kr >> 3;
#pragma unroll
      for (int it = 0; it < NQ; ++it) {
        const int idx = threadIdx.x + 256 * it;
        const int hh = idx / cq, c = idx - hh * cq;
        if (hh < 16) {
          const int head = g * 16 + hh;
          u32x4 v = {0u, 0u, 0u, 0u};
          if (head < H) v = *reinterpret_cast<const u32x4*>(q_lat + (size_t)head * ql_hs + (size_t)row * ql_ts + c * 8);
          *reinterpret_cast<u32x4*>(qs + (size_t)hh * DP + c * 8) = v;
        }
      }
    } else {
      for (int i = threadIdx.x; i < 16 * kr; i += 256) {
        const int hh = i / kr, e = i - hh * kr;
        const int head = g * 16 + hh;
        qs[(size_t)hh * DP + e] = head < H ? q_lat[(size_t)head * ql_hs + (size_t)row * ql_ts + e] : (uint16_t)0;
      }
    }
    // rotated part
#pragma unroll 4
    for (int i = threadIdx.x; i < 16 * rd; i += 256) {
      const int hh = i / rd, e2 = i - hh * rd;
      const int head = g * 16 + hh;
      uint16_t v = 0;
      if (head < H) {
        const uint16_t* qr = q + (size_t)row * q_stride + (size_t)head * (dim + rd) + dim;
        if (e2 < dims) {
          int k, partner;
          bool lead;                                  // the pair's first element
          if (interleaved) { k = e2 >> 1; partner = e2 ^ 1; lead = !(e2 & 1); }
          else { lead = e2 < half; k = lead ? e2 : e2 - half; partner = lead ? e2 + half : e2 - half; }
          const float a = bf16_to_f32(qr[e2]), b = bf16_to_f32(qr[partner]);
          const float c = cs[k], sn = cs[half + k];
          v = f32_to_bf16(lead ? a * c - b * sn : a * c + b * sn);
        } else {
          v = qr[e2];
        }
      }
      qs[(size_t)hh * DP + kr + e2] = v;
    }
  }
  __syncthreads();
  const uint16_t* qp = qs + (size_t)lr * DP + 4 * lg;   // this lane's operand of Q^T: head lr, dims 16 s + 4 lg .. + 3

  float m_run = -__builtin_inff(), l_run = 0.f;        // of head lr, over this wave's keys
  f32x4 acc[NM];                                       // O^T: latent dims 16 m + 4 lg + i of head lr
#pragma unroll
  for (int m = 0; m < NM; ++m) acc[m] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int ntiles = (pos - first + KT) / KT;
  const int tps = (ntiles + (int)gridDim.z - 1) / (int)gridDim.z;
  const int t_hi = min(ntiles, ((int)blockIdx.z + 1) * tps);
  const int cpr = D >> 3;                              // 16-byte chunks per cached row
  // A wave stages only its own 16 rows of a tile (nobody else reads them), so the waves run their tiles
  // without workgroup barriers, and the rows of tile t + 1 are loaded into registers before tile t is
  // computed: the loads' latency hides behind the MFMAs.
  constexpr int NLD = (16 * NDS * 2 + 63) / 64;        // 16-byte chunks per lane: 16 rows of at most NDS * 2 chunks
  u32x4 pre[NLD];
  // lane j < 16 resolves the cache slot of the wave's row j of a tile (-1: past the last key); the slots of
  // tile t + 1 are looked up while tile t's rows are fetched, so the page-table read is off the critical path
  auto slot_of = [&](int ti) {
    const int key = first + ti * KT + 16 * w + lane;
    int sl = -1;
    if (lane < 16 && ti < t_hi && key <= pos) sl = bt[key / bs] * bs + (key % bs);
    return sl;
  };
  int next_slot = slot_of(blockIdx.z * tps);
  auto issue = [&](int ti) {
    const int myslot = next_slot;
    next_slot = slot_of(ti + 1);
#pragma unroll
    for (int it = 0; it < NLD; ++it) {
      const int idx = lane + 64 * it;
      const int j = (int)__umulhi((unsigned)idx, cpr_magic), c = idx - j * cpr;     // idx / cpr (checked on the host)
      const int sl = __shfl(myslot, j & 15, 64);
      pre[it] = u32x4{0u, 0u, 0u, 0u};                 // rows past the last key are zero: 0 * stale bits could be NaN
      if (j < 16 && sl >= 0) pre[it] = *reinterpret_cast<const u32x4*>(cache + (long long)sl * D + c * 8);
    }
  };
  const int t_lo = blockIdx.z * tps;
  if (t_lo < t_hi) issue(t_lo);
  for (int ti = t_lo; ti < t_hi; ++ti) {
    const int k0 = first + ti * KT;
    const int n = min(KT, pos - k0 + 1);
#pragma unroll
    for (int it = 0; it < NLD; ++it) {
      const int idx = lane + 64 * it;
      const int j = (int)__umulhi((unsigned)idx, cpr_magic), c = idx - j * cpr;
      if (j < 16) *reinterpret_cast<u32x4*>(tile + (size_t)(16 * w + j) * DP + c * 8) = pre[it];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (ti + 1 < t_hi) issue(ti + 1);
    if (16 * w >= n) continue;                         // none of this wave's 16 keys exists (wave-uniform)
    // four independent accumulation chains (a chain of dependent MFMAs waits out each one's latency)
    f32x4 sp[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) sp[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    const uint16_t* kp = tile + (size_t)(16 * w + lr) * DP + 4 * lg;
#pragma unroll
    for (int s = 0; s < NDS; ++s) {
      if (s < nd) {
        const short4v a = *reinterpret_cast<const short4v*>(kp + 16 * s);
        const short4v b = *reinterpret_cast<const short4v*>(qp + 16 * s);
        sp[s & 3] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, sp[s & 3], 0, 0, 0);
      }
    }
    f32x4 sc;
#pragma unroll
    for (int i = 0; i < 4; ++i) sc[i] = (sp[0][i] + sp[1][i]) + (sp[2][i] + sp[3][i]);
    // sc[i]: key 16 w + 4 lg + i, head lr
    float mx = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sc[i] = (16 * w + 4 * lg + i < n) ? sc[i] * scale : -__builtin_inff();
      mx = fmaxf(mx, sc[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));            // key 16 w exists: finite
    const float m_new = fmaxf(m_run, mx);
    const float corr = expf(m_run - m_new);            // first tile: exp(-inf) = 0
    float p[4], sum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = expf(sc[i] - m_new);
      sum += p[i];
    }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    l_run = l_run * corr + sum;
    m_run = m_new;
    short4v pb;
#pragma unroll
    for (int i = 0; i < 4; ++i) pb[i] = (short)f32_to_bf16(p[i]);
    const bool rescale = __any(corr != 1.f);           // no head's maximum moved: the sums keep their scale
    const uint16_t* vp = tile + (size_t)(16 * w + 4 * lg) * DP + lr;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      if (m < nm) {
        short4v a;
#pragma unroll
        for (int j = 0; j < 4; ++j) a[j] = (short)vp[(size_t)j * DP + 16 * m];
        if (rescale) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[m][i] *= corr;
        }
        acc[m] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pb, acc[m], 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();                   // this tile's rows are read before the next ones land
  }
  // combine the four waves: every head's (max, sum) through LDS; O^T of waves 0 / 1 into two LDS buffers, waves
  // 2 / 3 added on top, and the output pass adds the two buffers
  __syncthreads();                                     // the last tile is fully read
  float* ml = reinterpret_cast<float*>(tile);          // [4 waves][16 heads][2], then [16 heads][2] combined
  const int ks = kr + 4;                               // padded: a head's rows start 4 banks apart
  float* os = ml + 160;                                // [2][16 heads][ks] fp32
  if (lg == 0) {
    ml[(w * 16 + lr) * 2] = m_run;
    ml[(w * 16 + lr) * 2 + 1] = l_run;
  }
  __syncthreads();
  float M = -__builtin_inff();
#pragma unroll
  for (int ww = 0; ww < 4; ++ww) M = fmaxf(M, ml[(ww * 16 + lr) * 2]);
  float Lsum = 0.f;
#pragma unroll
  for (int ww = 0; ww < 4; ++ww) {
    const float mw = ml[(ww * 16 + lr) * 2];
    Lsum += mw == -__builtin_inff() ? 0.f : ml[(ww * 16 + lr) * 2 + 1] * expf(mw - M);
  }
  const float f = m_run == -__builtin_inff() ? 0.f : expf(m_run - M);     // a wave (or a whole run) without keys adds nothing
  float* mine = os + (w & 1) * 16 * ks + lr * ks + 4 * lg;
#pragma unroll
  for (int ph = 0; ph < 2; ++ph) {
    if ((w >> 1) == ph) {
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        if (m < nm) {
          float4* dst = reinterpret_cast<float4*>(mine + 16 * m);
          float4 cur = ph == 0 ? make_float4(0.f, 0.f, 0.f, 0.f) : *dst;
          cur.x += acc[m][0] * f; cur.y += acc[m][1] * f; cur.z += acc[m][2] * f; cur.w += acc[m][3] * f;
          *dst = cur;
        }
      }
    }
    __syncthreads();
  }
  // 16 threads per head, four consecutive latent dims each
  const int hh = threadIdx.x >> 4, part = threadIdx.x & 15;
  const int head = g * 16 + hh;
  if (head >= H) return;
  // (M, Lsum) of head hh live in the lanes with lr == hh: lane hh of this thread's wave has them
  const float Mh = __shfl(M, hh, 64), Lh = __shfl(Lsum, hh, 64);
  const float* o0 = os + hh * ks;
  const float* o1 = o0 + 16 * ks;
  if (part_o) {
    const size_t slot = ((size_t)blockIdx.z * H + head) * rows + row;
    for (int e = part * 4; e < kr; e += 64) {
      const float4 x = *reinterpret_cast<const float4*>(o0 + e), y = *reinterpret_cast<const float4*>(o1 + e);
      *reinterpret_cast<float4*>(part_o + slot * kr + e) = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
    }
    if (part == 0) {
      part_ml[2 * slot] = Mh;
      part_ml[2 * slot + 1] = Lh;
    }
  } else {
    const float inv = 1.f / Lh;
    uint16_t* op = out + (size_t)head * o_hs + (size_t)row * o_ts;
    const bool ovec = ((uintptr_t)out & 7) == 0 && (o_hs & 3) == 0 && (o_ts & 3) == 0;
    for (int e = part * 4; e < kr; e += 64) {
      const float4 x = *reinterpret_cast<const float4*>(o0 + e), y = *reinterpret_cast<const float4*>(o1 + e);
      const float v0 = (x.x + y.x) * inv, v1 = (x.y + y.y) * inv, v2 = (x.z + y.z) * inv, v3 = (x.w + y.w) * inv;
      if (ovec) {
        *reinterpret_cast<uint2*>(op + e) = make_uint2(pack_bf16x2(v0, v1), pack_bf16x2(v2, v3));
      } else {
        op[e] = f32_to_bf16(v0); op[e + 1] = f32_to_bf16(v1); op[e + 2] = f32_to_bf16(v2); op[e + 3] = f32_to_bf16(v3);
      }
    }
  }
}

template <typename K>
int allow_lds(K kernel, size_t lds) {
  return (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
}

// LDS a workgroup may take: what the device reports, at most the 160 KB of a CDNA4 compute unit
size_t lds_max() {
  static size_t v = 0;
  if (!v) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || n <= 0)
      n = 64 * 1024;
    v = (size_t)n < 160 * 1024 ? (size_t)n : 160 * 1024;
  }
  return v;
}

template <typename T, bool VEC, int KT>
int launch(const void* q, int q_stride, const void* q_lat, long long ql_hs, long long ql_ts, const void* cache,
           const int* block_tables, int bt_stride, const int* cu_seqlens, int n_seqs, const int* positions, int rows, int H,
           int dim, int rd, int kr, int bs, float scale, int window, const float* cos_sin, int dims, int interleaved,
           void* out, long long o_hs, long long o_ts, int nw, int nsplit, float* part_o, float* part_ml, hipStream_t s) {
  constexpr int E = 16 / sizeof(T);
  const int D = kr + rd;
  const int DP = (D + E - 1) / E * E + E;           // padded row: 16-byte aligned, not a multiple of the bank span
  const int DQ = (D + 3) / 4 * 4;
  size_t lds;
  for (;; nw >>= 1) {
    lds = ((size_t)KT * DP * sizeof(T) + 3) / 4 * 4 + (size_t)nw * DQ * 4 + (size_t)nw * KT * 4;
    if (lds <= lds_max() || nw == 1) break;
  }
  if (lds > lds_max()) return -6;
  static int allowed = -1;                           // once per kernel instance
  if (allowed != 0 && lds > 64 * 1024) {
    allowed = allow_lds(latent_attn_rows_kernel<T, VEC, KT>, lds_max());
    if (allowed != 0) return allowed;
  }
  const dim3 grid(rows, (H + nw - 1) / nw, nsplit);
  latent_attn_rows_kernel<T, VEC, KT><<<grid, 64 * nw, lds, s>>>(
      (const T*)q, q_stride, (const T*)q_lat, ql_hs, ql_ts, (const T*)cache, block_tables, bt_stride, cu_seqlens, n_seqs,
      positions, H, dim, rd, kr, bs, scale, window, cos_sin, dims, interleaved, (T*)out, o_hs, o_ts, DP, DQ,
      nsplit > 1 ? part_o : nullptr, part_ml);
  if (nsplit > 1)
    latent_attn_reduce_kernel<T><<<dim3(rows, H), kr >= 256 ? 256 : 64, 0, s>>>(part_o, part_ml, nsplit, kr, (T*)out, o_hs, o_ts);
  return 0;
}


template <int NM, int NDS>
int launch_mfma(const void* q, int q_stride, const void* q_lat, long long ql_hs, long long ql_ts, const void* cache,
                const int* block_tables, int bt_stride, const int* cu_seqlens, int n_seqs, const int* positions, int rows,
                int H, int dim, int rd, int kr, int bs, float scale, int window, const float* cos_sin, int dims,
                int interleaved, void* out, long long o_hs, long long o_ts, int nsplit, float* part_o, float* part_ml,
                hipStream_t s) {
  const int D = kr + rd;
  const int DP = D + 8;                                // rows 16-byte aligned, consecutive rows 4 banks apart
  // idx / cpr for idx < 16 * cpr + 64 as a multiply-high (cpr = 16-byte chunks per cached row)
  const unsigned cpr = (unsigned)D >> 3;
  const unsigned magic = (unsigned)((0x100000000ull + cpr - 1) / cpr);
  for (unsigned i = 0; i < 16 * cpr + 64; ++i)
    if ((unsigned)(((unsigned long long)i * magic) >> 32) != i / cpr) return -9;
  const size_t lds = (size_t)16 * DP * 2 + std::max((size_t)64 * DP * 2, (size_t)(160 + 32 * (kr + 4)) * 4);     // queries; tiles, then the combine buffers
  if (lds > lds_max()) return -6;
  static int allowed = -1;
  if (allowed != 0 && lds > 64 * 1024) {
    allowed = allow_lds(latent_attn_mfma_kernel<NM, NDS>, lds_max());
    if (allowed != 0) return allowed;
  }
  latent_attn_mfma_kernel<NM, NDS><<<dim3(rows, (H + 15) / 16, nsplit), 256, lds, s>>>(
      (const uint16_t*)q, q_stride, (const uint16_t*)q_lat, ql_hs, ql_ts, (const uint16_t*)cache, block_tables, bt_stride,
      cu_seqlens, n_seqs, positions, H, dim, rd, kr, bs, scale, window, cos_sin, dims, interleaved, DP, (uint16_t*)out, o_hs,
      o_ts, nsplit > 1 ? part_o : nullptr, part_ml, magic);
  if (nsplit > 1)
    latent_attn_reduce_kernel<uint16_t><<<dim3(rows, H), kr >= 256 ? 256 : 64, 0, s>>>(part_o, part_ml, nsplit, kr,
                                                                                      (uint16_t*)out, o_hs, o_ts);
  return 0;
}

}  // namespace

// q [rows, H * (dim + rd)] (row stride q_stride); q_lat / out [H, rows, kr] with their own head and row strides;
// cache [NB, 1, bs, kr + rd]; cu_seqlens (n_seqs + 1 row offsets) maps rows to block-table rows, nullptr: row i
// uses table row i.  Workgroups are sized so that the grid covers the chip where the step allows; nsplit > 1 cuts
// every row's keys into that many runs (steps of few rows over long contexts) whose partial results, in
// part_o [nsplit, H, rows, kr] and part_ml [nsplit, H, rows, 2] (fp32), a second kernel combines.
extern "C" int dgi_latent_attn_rows(const void* q, int q_stride, const void* q_lat, long long ql_hs, long long ql_ts,
                                    const void* cache, const int* block_tables, int bt_stride, const int* cu_seqlens,
                                    int n_seqs, const int* positions, int rows, int H, int dim, int rd, int kr,
                                    int block_size, float scale, int window, const float* cos_sin, int dims,
                                    int interleaved, void* out, long long o_hs, long long o_ts, int is_f32, int nsplit,
                                    float* part_o, float* part_ml, int mfma, hipStream_t s) {
  if (rows == 0) return 0;
  if (H <= 0 || kr <= 0 || rd < 0 || dim < 0 || window < 0) return -2;
  if (nsplit < 1 || nsplit > 65535 || (nsplit > 1 && (!part_o || !part_ml)) || H > 65535) return -7;
  if (mfma) {
    if (is_f32 || kr % 16 || (kr + rd) % 16 || kr > 512 || kr + rd > 576 || ((uintptr_t)cache & 15)) return -8;
    if (dims > rd || (dims & 1) || (dims > 0 && !cos_sin)) return -3;
    int rc;
    if (kr <= 128 && kr + rd <= 192)
      rc = launch_mfma<8, 12>(q, q_stride, q_lat, ql_hs, ql_ts, cache, block_tables, bt_stride, cu_seqlens, n_seqs, positions,
                              rows, H, dim, rd, kr, block_size, scale, window, cos_sin, dims, interleaved, out, o_hs, o_ts,
                              nsplit, part_o, part_ml, s);
    else
      rc = launch_mfma<32, 36>(q, q_stride, q_lat, ql_hs, ql_ts, cache, block_tables, bt_stride, cu_seqlens, n_seqs, positions,
                               rows, H, dim, rd, kr, block_size, scale, window, cos_sin, dims, interleaved, out, o_hs, o_ts,
                               nsplit, part_o, part_ml, s);
    if (rc != 0) return rc;
    DGI_CHECK_LAUNCH();
    return 0;
  }
  if (dims > rd || (dims & 1) || (dims > 0 && !cos_sin)) return -3;
  if (H > 65535 * 16) return -4;
  const int E = is_f32 ? 4 : 8;
  const bool vec = kr % E == 0 && (kr + rd) % E == 0 && ((uintptr_t)cache & 15) == 0;
  if (kr > (vec ? 64 * E * (is_f32 ? 4 : 2) : 64 * 8)) return -5;
  // heads per workgroup: as many as share a staged tile, fewer when the step has too few rows to fill the chip
  int nw = 16;
  while (nw > 1 && nw / 2 >= H) nw >>= 1;
  while (nw > 2 && (long long)rows * ((H + nw - 1) / nw) * nsplit < 512) nw >>= 1;
  int rc;
#define DGI_LA(TT_, VV_, KK_)                                                                                       \
  rc = launch<TT_, VV_, KK_>(q, q_stride, q_lat, ql_hs, ql_ts, cache, block_tables, bt_stride, cu_seqlens, n_seqs, \
                             positions, rows, H, dim, rd, kr, block_size, scale, window, cos_sin, dims, interleaved, \
                             out, o_hs, o_ts, nw, nsplit, part_o, part_ml, s)
  if (is_f32) { if (vec) DGI_LA(float, true, 32); else DGI_LA(float, false, 32); }
  else { if (vec) DGI_LA(uint16_t, true, 64); else DGI_LA(uint16_t, false, 64); }
#undef DGI_LA
  if (rc != 0) return rc;
  DGI_CHECK_LAUNCH();
  return 0;
}
