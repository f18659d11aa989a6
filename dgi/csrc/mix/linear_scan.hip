// dgi/csrc/mix/linear_scan.hip — mixers that carry a matrix state S [dk, dv] per (sequence, head) from
// token to token, and the small row kernels around them.
//
//   linear_scan      the recurrence over packed rows (decode rows and prompt portions alike), three updates:
//                      wkv    o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T,  w = exp(-exp(w_raw + w0))
//                      delta  S <- g S;  S += k (beta (v - S^T k))^T;  o = S^T q   (q, k unit vectors, q * dk^-1/2)
//                             g = exp(-exp(a_log) softplus(a_raw + dt_bias)),  beta = sigmoid(b_raw)
//                      mlstm  m' = max(f + m, i);  S <- e^(f+m-m') S + e^(i-m') k v^T  (n likewise, k alone);
//                             o = S^T q' / (max(|n . q'|, e^-m') + 1e-6),  q' = q dk^-1/2,
//                             i = cap tanh(i_raw / cap),  f = logsigmoid(cap tanh(f_raw / cap))
//   token_shift      n blends h + (h' - h) mu of a row with the previous token's row (state slot at a portion's start)
//   head_norm_gate   per-head RMS norm of the recurrence's output, weight, silu / sigmoid gate
//   rms_pair_mean    0.5 (a / rms(a) wa + b / rms(b) wb) over the model width
//
// linear_scan layout.  A workgroup (256 threads) owns (sequence, head, CB value columns).  Inside a wave,
// lane = j * KS + s: column j of the wave's CW = 64 / KS columns, key slice s of KS slices; a thread keeps R
// consecutive key channels of its column in registers (KS * R >= dk), so a token costs R fused multiply-adds
// per pass and the sums over the key dimension finish with log2(KS) xor-shuffles between ADJACENT lanes
// (constant offsets below 16) — no barrier per token.  Tokens are staged TT (16) at a time: the tile is
// loaded into registers, spread over all threads, while the previous tile is computed, then goes to LDS
// (slices padded apart so the KS broadcast reads of a wave hit different banks; 16-byte reads).  Per-token
// scalars are computed once per tile in parallel: unit norms / the bonus dot product by sixteen lanes per
// token, decays and gates by one lane per token from gate inputs staged with the tile; only the stabiliser's
// running maximum is a serial pass of one thread (adds and maxima; its exponentials are parallel again).
// The token loop reads LDS only.  Everything is fp32; q / k / v arrive as bf16 or fp32.
// A portion that starts at position 0 reads no state; the state is written back at the end of the portion.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

constexpr int WKV = 0, DELTA = 1, MLSTM = 2;
constexpr int TT = 8;            // tokens per staged tile

struct ScanArgs {
  float* y;                      // [T, H * dv]
  const void *q, *k, *v;         // rows with their own strides (elements); q: the receptance for wkv
  int q_stride, k_stride, v_stride;
  const float *aux1, *aux2;      // per token: w_raw [T, H*dk] | b_raw [T, H] | i_raw [T, H];  - | a_raw | f_raw
  int aux1_stride, aux2_stride;
  const float *par1, *par2;      // w0 [H*dk] | a_log [H] | -;   u [H*dk] | dt_bias [H] | -
  float* state;                  // [slots, H, dk, dv]
  float* norm;                   // mlstm: [slots, H, dk]
  float* mx;                     // mlstm: [slots, H]
  float *norm_new, *mx_new;      // mlstm with several column blocks per head: [n_seq, H, dk] / [n_seq, H] staging (see below)
  const int *positions, *seq_row0, *seq_slots;
  int H, G, dk, dv;
  int KS, CW, nwc, CB;           // key slices per wave, columns per wave, computing waves, columns per workgroup
  float cap;
};

// Sums inside the vector ALU (data-parallel-primitive moves) instead of __shfl_xor, which goes through the LDS permute
// unit: the sums sit on the token loop's dependent chain.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
// total over the KS adjacent lanes (aligned group, KS a power of two up to 16) that hold the slices of one column
template <int KS>
__device__ __forceinline__ float slice_sum(float v) {
  if constexpr (KS >= 2) v += dpp_move<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  if constexpr (KS >= 4) v += dpp_move<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  if constexpr (KS >= 8) v += dpp_move<0x141>(v);     // mirror inside each half row: the other quad's total
  if constexpr (KS >= 16) v += dpp_move<0x140>(v);    // mirror inside the row: the other half's total
  return v;
}
// total over a row of sixteen lanes, in every lane (four rotate-adds)
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_move<0x128>(v);
  v += dpp_move<0x124>(v);
  v += dpp_move<0x122>(v);
  v += dpp_move<0x121>(v);
  return v;
}

__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float logsigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// R key channels per thread, KS key slices per value column (adjacent lanes: lane = column * KS + slice, so the sums
// over the key dimension are log2(KS) xor-shuffles with constant offsets below 16), TT tokens per staged tile.
template <int MODE, typename TI, int R, int KS, int TT>
__global__ __launch_bounds__(256) void linear_scan_kernel(const ScanArgs a) {
  constexpr int CW = 64 / KS;                      // value columns per wave
  constexpr int RP = R + 4;                        // padded key slice in LDS
  constexpr int KP = KS * RP;                      // padded key row
  constexpr int KSR = KS * R;                      // key channels covered (>= dk)
  constexpr int NT = 256;
  constexpr int NPF = (TT * KSR + NT - 1) / NT;    // staged key elements per thread and tile
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int seq = blockIdx.x, head = blockIdx.y, cblk = blockIdx.z;
  const int row0 = a.seq_row0[seq], n = a.seq_row0[seq + 1] - row0;
  if (n <= 0) return;
  const int p0 = a.positions[row0], slot = a.seq_slots[seq];
  const int dk = a.dk, dv = a.dv, H = a.H;
  const int kvh = head / (H / a.G);
  const int CB = a.CB;
  const int NPV = (TT * CB + NT - 1) / NT;         // staged value elements per thread and tile (CB <= 256: at most TT)
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int s = lane % KS, jl = lane / KS;
  const bool computes = wave < a.nwc;
  const int cl = wave * CW + jl;                   // column inside the workgroup
  const int col = cblk * CB + cl;
  const bool col_ok = computes && col < dv;
  constexpr int NV = MODE == WKV ? 3 : 2;
  float* sk = sm;                                  // [TT][KP]
  float* sq = sk + TT * KP;
  float* sw = sq + TT * KP;                        // wkv only
  float* sv = sm + NV * TT * KP;                   // [TT][CB]
  float* sc = sv + TT * CB;                        // [TT][4] per-token scalars
  float* sg = sc + TT * 4;                         // [TT][4] raw gate inputs / stabiliser scratch
  float* su = sg + TT * 4;                         // wkv: [KP] bonus

  float S[R], N[MODE == MLSTM ? R : 1];
  const size_t sbase = ((size_t)slot * H + head) * dk;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int ch = s * R + i;
    S[i] = (p0 > 0 && col_ok && ch < dk) ? a.state[(sbase + ch) * dv + col] : 0.f;
    if constexpr (MODE == MLSTM) N[i] = (p0 > 0 && computes && ch < dk) ? a.norm[sbase + ch] : 0.f;
  }
  float m_run = 0.f;                               // mlstm stabiliser, carried by thread 0
  if (MODE == MLSTM && tid == 0 && p0 > 0) m_run = a.mx[(size_t)slot * H + head];
  if constexpr (MODE == WKV) {
    for (int ch = tid; ch < KSR; ch += NT) su[(ch / R) * RP + (ch % R)] = ch < dk ? a.par2[head * dk + ch] : 0.f;
  }

  const TI* qp = (const TI*)a.q + (size_t)kvh * dk;
  const TI* kp = (const TI*)a.k + (size_t)kvh * dk;
  const TI* vp = (const TI*)a.v + (size_t)head * dv + cblk * CB;
  float pk[NPF], pq[NPF], pw[MODE == WKV ? NPF : 1], pv[TT], pg1 = 0.f, pg2 = 0.f;
  auto load_tile = [&](int t0) {
#pragma unroll
    for (int m = 0; m < NPF; ++m) {
      const int e = tid + m * NT;
      const int tt = e / KSR, ch = e % KSR;
      const bool ok = tt < TT && t0 + tt < n && ch < dk;
      const size_t row = (size_t)(row0 + t0 + tt);
      pk[m] = ok ? ldf<TI>(kp + row * a.k_stride + ch) : 0.f;
      pq[m] = ok ? ldf<TI>(qp + row * a.q_stride + ch) : 0.f;
      if constexpr (MODE == WKV)
        pw[m] = ok ? expf(-expf(a.aux1[row * a.aux1_stride + head * dk + ch] + a.par1[head * dk + ch])) : 0.f;
    }
#pragma unroll
    for (int m = 0; m < TT; ++m) {
      pv[m] = 0.f;
      if (m < NPV) {
        const int e = tid + m * NT;
        const int tt = e / CB, c = e - tt * CB;
        if (tt < TT && t0 + tt < n && cblk * CB + c < dv) pv[m] = ldf<TI>(vp + (size_t)(row0 + t0 + tt) * a.v_stride + c);
      }
    }
    if (MODE != WKV && tid < TT && t0 + tid < n) {
      const size_t row = (size_t)(row0 + t0 + tid);
      pg1 = a.aux1[row * a.aux1_stride + head];
      pg2 = a.aux2[row * a.aux2_stride + head];
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int m = 0; m < NPF; ++m) {
      const int e = tid + m * NT;
      const int tt = e / KSR, ch = e % KSR;
      if (tt < TT) {
        const int o = tt * KP + (ch / R) * RP + (ch % R);
        sk[o] = pk[m];
        sq[o] = pq[m];
        if constexpr (MODE == WKV) sw[o] = pw[m];
      }
    }
#pragma unroll
    for (int m = 0; m < TT; ++m) {
      if (m < NPV) {
        const int e = tid + m * NT;
        if (e < TT * CB) sv[e] = pv[m];
      }
    }
    if (MODE != WKV && tid < TT) {
      sg[tid * 4] = pg1;
      sg[tid * 4 + 1] = pg2;
    }
  };
  const float qscale = 1.f / sqrtf((float)dk);

  load_tile(0);
  for (int t0 = 0; t0 < n; t0 += TT) {
    const int nt = min(TT, n - t0);
    store_tile();
    __syncthreads();
    // ---- per-token scalars
    if constexpr (MODE == MLSTM) {
      // gates in parallel, the running maximum serially (adds and maxima only), the exponentials in parallel again
      if (tid < nt) {
        sg[tid * 4 + 2] = a.cap * tanhf(sg[tid * 4] / a.cap);
        sg[tid * 4 + 3] = logsigmoid_f(a.cap * tanhf(sg[tid * 4 + 1] / a.cap));
      }
      __syncthreads();
      if (tid == 0) {
        for (int tt = 0; tt < nt; ++tt) {
          const float m_new = fmaxf(sg[tt * 4 + 3] + m_run, sg[tt * 4 + 2]);
          sg[tt * 4] = m_run;                       // the maximum before this token
          sg[tt * 4 + 1] = m_new;
          m_run = m_new;
        }
      }
      __syncthreads();
      if (tid < nt) {
        const float m_old = sg[tid * 4], m_new = sg[tid * 4 + 1];
        sc[tid * 4 + 0] = expf(sg[tid * 4 + 3] + m_old - m_new);
        sc[tid * 4 + 1] = expf(sg[tid * 4 + 2] - m_new);
        sc[tid * 4 + 2] = expf(-m_new);
      }
    } else {
      // sixteen lanes per token: sums over the key channels, four shuffles inside the group
      const int l = tid & 15;
      for (int tt = tid >> 4; tt < nt; tt += NT / 16) {
        float r1 = 0.f, r2 = 0.f;
        for (int i = l; i < dk; i += 16) {
          const int pi = (i / R) * RP + (i % R);
          const float kv = sk[tt * KP + pi], qv = sq[tt * KP + pi];
          if (MODE == WKV) {
            r1 += qv * kv * su[pi];                 // the bonus: sum_i r_i u_i k_i
          } else {
            r1 += kv * kv;
            r2 += qv * qv;
          }
        }
        r1 = row16_sum(r1);
        if (MODE == DELTA) r2 = row16_sum(r2);
        if (l == 0) {
          if (MODE == WKV) {
            sc[tt * 4] = r1;
          } else {
            const float dt = softplus_f(sg[tt * 4 + 1] + a.par2[head]);
            sc[tt * 4 + 0] = expf(-expf(a.par1[head]) * dt);                        // decay
            sc[tt * 4 + 1] = 1.f / (1.f + expf(-sg[tt * 4]));                       // write strength
            sc[tt * 4 + 2] = 1.f / sqrtf(r1 + 1e-6f);                               // 1 / |k|
            sc[tt * 4 + 3] = qscale / sqrtf(r2 + 1e-6f);                            // dk^-1/2 / |q|
          }
        }
      }
    }
    __syncthreads();
    if (t0 + TT < n) load_tile(t0 + TT);             // in flight while this tile is computed
    if (computes) {
      // four tokens per trip, free of branches (the outputs wait in registers and are stored after the trip), so the
      // LDS reads of the later tokens are issued under the arithmetic of the earlier ones
      auto token = [&](int tt) -> float {
        const float4* kk = reinterpret_cast<const float4*>(sk + tt * KP + s * RP);
        const float4* qq = reinterpret_cast<const float4*>(sq + tt * KP + s * RP);
        const float vj = sv[tt * CB + cl];
        float o;
        if constexpr (MODE == WKV) {
          const float4* ww = reinterpret_cast<const float4*>(sw + tt * KP + s * RP);
          float acc = 0.f;
#pragma unroll
          for (int i = 0; i < R / 4; ++i) {
            const float4 q4 = qq[i], k4 = kk[i], w4 = ww[i];
            acc += S[4 * i] * q4.x + S[4 * i + 1] * q4.y + S[4 * i + 2] * q4.z + S[4 * i + 3] * q4.w;
            S[4 * i] = w4.x * S[4 * i] + k4.x * vj;
            S[4 * i + 1] = w4.y * S[4 * i + 1] + k4.y * vj;
            S[4 * i + 2] = w4.z * S[4 * i + 2] + k4.z * vj;
            S[4 * i + 3] = w4.w * S[4 * i + 3] + k4.w * vj;
          }
          acc = slice_sum<KS>(acc);
          o = acc + sc[tt * 4] * vj;
        } else if constexpr (MODE == DELTA) {
          const float g = sc[tt * 4], beta = sc[tt * 4 + 1], rk = sc[tt * 4 + 2], rq = sc[tt * 4 + 3];
          float pred = 0.f;
#pragma unroll
          for (int i = 0; i < R / 4; ++i) {
            const float4 k4 = kk[i];
            pred += S[4 * i] * k4.x + S[4 * i + 1] * k4.y + S[4 * i + 2] * k4.z + S[4 * i + 3] * k4.w;
          }
          pred = slice_sum<KS>(pred);
          const float ku = beta * (vj - pred * g * rk) * rk;
          float acc = 0.f;
#pragma unroll
          for (int i = 0; i < R / 4; ++i) {
            const float4 k4 = kk[i], q4 = qq[i];
            S[4 * i] = g * S[4 * i] + k4.x * ku;
            S[4 * i + 1] = g * S[4 * i + 1] + k4.y * ku;
            S[4 * i + 2] = g * S[4 * i + 2] + k4.z * ku;
            S[4 * i + 3] = g * S[4 * i + 3] + k4.w * ku;
            acc += S[4 * i] * q4.x + S[4 * i + 1] * q4.y + S[4 * i + 2] * q4.z + S[4 * i + 3] * q4.w;
          }
          acc = slice_sum<KS>(acc);
          o = acc * rq;
        } else {
          const float fa = sc[tt * 4], fb = sc[tt * 4 + 1], em = sc[tt * 4 + 2];
          const float bv = fb * vj;
          float acc = 0.f, nq = 0.f;
#pragma unroll
          for (int i = 0; i < R / 4; ++i) {
            const float4 k4 = kk[i], q4 = qq[i];
            const float kx[4] = {k4.x, k4.y, k4.z, k4.w}, qx[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              S[4 * i + j] = fa * S[4 * i + j] + kx[j] * bv;
              acc += S[4 * i + j] * qx[j];
              N[4 * i + j] = fa * N[4 * i + j] + fb * kx[j];
              nq += N[4 * i + j] * qx[j];
            }
          }
          acc = slice_sum<KS>(acc);
          nq = slice_sum<KS>(nq);
          o = acc * qscale / (fmaxf(fabsf(nq * qscale), em) + 1e-6f);
        }
        return o;
      };
      const size_t ys = (size_t)H * dv;
      float* yp = a.y + (size_t)(row0 + t0) * ys + (size_t)head * dv + col;
      int tt = 0;
      for (; tt + 4 <= nt; tt += 4) {
        const float o0 = token(tt), o1 = token(tt + 1), o2 = token(tt + 2), o3 = token(tt + 3);
        if (s == 0 && col_ok) {
          yp[tt * ys] = o0;
          yp[(tt + 1) * ys] = o1;
          yp[(tt + 2) * ys] = o2;
          yp[(tt + 3) * ys] = o3;
        }
      }
      for (; tt < nt; ++tt) {
        const float o = token(tt);
        if (s == 0 && col_ok) yp[tt * ys] = o;
      }
    }
    __syncthreads();                                 // the tile is consumed before the next one overwrites it
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int ch = s * R + i;
    if (col_ok && ch < dk) a.state[(sbase + ch) * dv + col] = S[i];
    if constexpr (MODE == MLSTM) {
      // every column block of a head reads the normaliser and the maximum at its start and block 0 writes them at
      // its end: with several blocks per head the new values go to a staging row and a second launch commits them,
      // so a block that starts late still reads the old state
      if (cblk == 0 && wave == 0 && jl == 0 && ch < dk) {
        if (a.norm_new) a.norm_new[((size_t)seq * H + head) * dk + ch] = N[i];
        else a.norm[sbase + ch] = N[i];
      }
    }
  }
  if (MODE == MLSTM && cblk == 0 && tid == 0) {
    if (a.mx_new) a.mx_new[(size_t)seq * H + head] = m_run;
    else a.mx[(size_t)slot * H + head] = m_run;
  }
}

// second launch of a matrix-memory scan whose heads span several column blocks: staged normaliser / maximum -> slots
__global__ __launch_bounds__(256) void mlstm_commit_kernel(float* __restrict__ norm, float* __restrict__ mx,
                                                           const float* __restrict__ norm_new,
                                                           const float* __restrict__ mx_new,
                                                           const int* __restrict__ seq_row0,
                                                           const int* __restrict__ seq_slots, int H, int dk) {
  const int seq = blockIdx.x;
  if (seq_row0[seq + 1] <= seq_row0[seq]) return;
  const size_t slot = (size_t)seq_slots[seq];
  for (int i = threadIdx.x; i < H * dk; i += blockDim.x) norm[slot * H * dk + i] = norm_new[(size_t)seq * H * dk + i];
  for (int i = threadIdx.x; i < H; i += blockDim.x) mx[slot * H + i] = mx_new[(size_t)seq * H + i];
}

template <int MODE, typename TI, int R, int KS, int TT>
int launch_scan_one(const ScanArgs& a, dim3 grid, hipStream_t st) {
  constexpr int NV = MODE == WKV ? 3 : 2;
  constexpr int KP = KS * (R + 4);
  const size_t lds = (size_t)(NV * TT * KP + TT * a.CB + 8 * TT + (MODE == WKV ? KP : 0)) * sizeof(float);
  if (lds > 64 * 1024) return -6;
  linear_scan_kernel<MODE, TI, R, KS, TT><<<grid, 256, lds, st>>>(a);
  return 0;
}

// short: a step of (nearly) single rows per sequence, i.e. decode: tiles of 4 tokens keep the staging registers few, so
// more workgroups fit a compute unit and the step streams the states at a higher rate; prompt portions take 16-token tiles
template <int MODE, typename TI>
int launch_scan(const ScanArgs& a, int R, bool short_rows, dim3 grid, hipStream_t st) {
  if (R == 32) return short_rows ? launch_scan_one<MODE, TI, 32, 16, 4>(a, grid, st) : launch_scan_one<MODE, TI, 32, 16, 8>(a, grid, st);
  if (R == 4 && a.KS == 16) return launch_scan_one<MODE, TI, 4, 16, 16>(a, grid, st);
  if (R == 8 && a.KS == 8) return launch_scan_one<MODE, TI, 8, 8, 16>(a, grid, st);
  if (R == 8 && a.KS == 16) return launch_scan_one<MODE, TI, 8, 16, 16>(a, grid, st);
  if (R != 16) return -5;
#define DGI_KS(K_, T_) return short_rows ? launch_scan_one<MODE, TI, 16, K_, 4>(a, grid, st) : launch_scan_one<MODE, TI, 16, K_, T_>(a, grid, st)
  switch (a.KS) {
    case 1: DGI_KS(1, 16);
    case 2: DGI_KS(2, 16);
    case 4: DGI_KS(4, 16);
    case 8: DGI_KS(8, 16);
    case 16: DGI_KS(16, 8);
  }
#undef DGI_KS
  return -5;
}

// ---------------------------------------------------------------------------------------------
template <typename TH, typename TO>
__global__ __launch_bounds__(256) void token_shift_kernel(TO* __restrict__ out, const TH* __restrict__ h, int h_stride,
                                                          const float* __restrict__ mu, int nmix,
                                                          const float* __restrict__ tail, const int* __restrict__ positions,
                                                          const int* __restrict__ row_seq, const int* __restrict__ seq_row0,
                                                          const int* __restrict__ seq_slots, int T, int W) {
  const int t = blockIdx.x;
  const int seq = row_seq[t];
  const bool first = t == seq_row0[seq];
  const bool start = first && positions[t] == 0;
  const TH* cur = h + (size_t)t * h_stride;
  const TH* prev_row = first ? nullptr : h + (size_t)(t - 1) * h_stride;
  const float* prev_tail = (first && !start) ? tail + (size_t)seq_slots[seq] * W : nullptr;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float x = ldf<TH>(cur + c);
    const float p = prev_row ? ldf<TH>(prev_row + c) : (prev_tail ? prev_tail[c] : 0.f);
    for (int m = 0; m < nmix; ++m)
      stf<TO>(out + ((size_t)m * T + t) * W + c, x + (p - x) * mu[(size_t)m * W + c]);
  }
}

// after token_shift_kernel (same stream): every portion's last row becomes the slot's previous input
template <typename TH>
__global__ __launch_bounds__(256) void token_shift_tail_kernel(const TH* __restrict__ h, int h_stride,
                                                               float* __restrict__ tail, const int* __restrict__ seq_row0,
                                                               const int* __restrict__ seq_slots, int W) {
  const int seq = blockIdx.x;
  const int r1 = seq_row0[seq + 1];
  if (r1 <= seq_row0[seq]) return;
  const TH* last = h + (size_t)(r1 - 1) * h_stride;
  float* dst = tail + (size_t)seq_slots[seq] * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) dst[c] = ldf<TH>(last + c);
}

// one wave per (row, head): y / rms(y) over the head's dv columns, times w, times silu(z) or sigmoid(z)
template <typename TZ, typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(TO* __restrict__ out, const float* __restrict__ y,
                                                             const TZ* __restrict__ z, int z_stride,
                                                             const float* __restrict__ w, int wlen, int T, int H, int dv,
                                                             float eps, int sigmoid_gate) {
  const long long unit = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= (long long)T * H) return;
  const int t = (int)(unit / H), head = (int)(unit - (long long)t * H);
  const int lane = threadIdx.x & 63;
  const float* yp = y + ((size_t)t * H + head) * dv;
  float ss = 0.f;
  for (int d = lane; d < dv; d += 64) ss += yp[d] * yp[d];
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)dv + eps);
  const TZ* zp = z + (size_t)t * z_stride + (size_t)head * dv;
  TO* op = out + ((size_t)t * H + head) * dv;
  for (int d = lane; d < dv; d += 64) {
    const float g = ldf<TZ>(zp + d);
    const float sg = 1.f / (1.f + expf(-g));
    stf<TO>(op + d, yp[d] * inv * w[(head * dv + d) % wlen] * (sigmoid_gate ? sg : g * sg));
  }
}


template <typename T> __device__ __forceinline__ void ld4v(const T* p, float* f);
template <> __device__ __forceinline__ void ld4v<uint16_t>(const uint16_t* p, float* f) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
}
template <> __device__ __forceinline__ void ld4v<float>(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
template <typename T> __device__ __forceinline__ void st4v(T* p, const float* f);
template <> __device__ __forceinline__ void st4v<float>(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
}
template <> __device__ __forceinline__ void st4v<uint16_t>(uint16_t* p, const float* f) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]));
}

// Sixteen lanes per (row, head), four columns per access (dv a multiple of 4, at most 256): the head's values stay in
// registers between the sum of squares (four rotate-adds inside the row of lanes) and the store.
template <typename TZ, typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_vec_kernel(TO* __restrict__ out, const float* __restrict__ y,
                                                                 const TZ* __restrict__ z, int z_stride,
                                                                 const float* __restrict__ w, int wlen, int T, int H, int dv,
                                                                 float eps, int sigmoid_gate) {
  constexpr int MAXCH = 4;
  const long long unit = (long long)blockIdx.x * 16 + (threadIdx.x >> 4);
  const bool live = unit < (long long)T * H;
  const int t = live ? (int)(unit / H) : 0, head = live ? (int)(unit - (long long)t * H) : 0;
  const int l = threadIdx.x & 15;
  const float* yp = y + ((size_t)t * H + head) * dv;
  float v[MAXCH][4];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < MAXCH; ++k) {
    const int c = (l + 16 * k) * 4;
    if (live && c < dv) {
      ld4v<float>(yp + c, v[k]);
      ss += v[k][0] * v[k][0] + v[k][1] * v[k][1] + v[k][2] * v[k][2] + v[k][3] * v[k][3];
    }
  }
  const float inv = 1.f / sqrtf(row16_sum(ss) / (float)dv + eps);
  if (!live) return;
  const TZ* zp = z + (size_t)t * z_stride + (size_t)head * dv;
  TO* op = out + ((size_t)t * H + head) * dv;
#pragma unroll
  for (int k = 0; k < MAXCH; ++k) {
    const int c = (l + 16 * k) * 4;
    if (c < dv) {
      float g[4], wv[4], o[4];
      ld4v<TZ>(zp + c, g);
      ld4v<float>(w + (head * dv + c) % wlen, wv);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float sg = 1.f / (1.f + expf(-g[j]));
        o[j] = v[k][j] * inv * wv[j] * (sigmoid_gate ? sg : g[j] * sg);
      }
      st4v<TO>(op + c, o);
    }
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void rms_pair_mean_kernel(float* __restrict__ out, const TA* __restrict__ a, int a_stride,
                                                            const TA* __restrict__ b, int b_stride,
                                                            const float* __restrict__ wa, const float* __restrict__ wb,
                                                            int W, float eps) {
  __shared__ float red[8];
  const int t = blockIdx.x;
  const TA* ap = a + (size_t)t * a_stride;
  const TA* bp = b + (size_t)t * b_stride;
  float sa = 0.f, sb = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float x = ldf<TA>(ap + c), y = ldf<TA>(bp + c);
    sa += x * x;
    sb += y * y;
  }
  sa = wave_sum(sa);
  sb = wave_sum(sb);
  if ((threadIdx.x & 63) == 0) {
    red[threadIdx.x >> 6] = sa;
    red[4 + (threadIdx.x >> 6)] = sb;
  }
  __syncthreads();
  const float ia = 0.5f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)W + eps);
  const float ib = 0.5f / sqrtf((red[4] + red[5] + red[6] + red[7]) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256)
    out[(size_t)t * W + c] = ldf<TA>(ap + c) * ia * wa[c] + ldf<TA>(bp + c) * ib * wb[c];
}

}  // namespace

// value columns of one workgroup with KS lanes per column: up to four waves of 64 / KS columns
static int scan_columns(int KS, int dv) {
  const int CW = 64 / KS;
  int nwc = (dv + CW - 1) / CW;
  if (nwc > 4) nwc = 4;
  return nwc * CW;
}

// Key channels per thread.  A decode-shaped step streams the states: 16 channels per thread, all columns of a head in
// one workgroup.  A prompt portion is a dependent chain per (sequence, head, column) whose length per token grows with
// the channels a thread holds, so while the grid stays within two workgroups per compute unit a head is spread over
// more lanes per column (and so over more workgroups): 4 or 8 channels per thread.  Beyond that the step is bound by
// the instructions issued, and the wide layout issues the fewest.
static int scan_channels(int dk, int dv, int H, int n_seq, int rows) {
  if (dk > 256) return 32;
  if (rows <= 4 * n_seq) return 16;
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    return n > 0 ? n : 256;
  }();
  for (int R = 4; R <= 8; R *= 2) {
    int KS = 1;
    while (KS * R < dk) KS <<= 1;
    if (!((R == 4 && KS == 16) || (R == 8 && (KS == 8 || KS == 16)))) continue;      // the layouts instantiated
    const int CB = scan_columns(KS, dv);
    const long grid = (long)n_seq * H * ((dv + CB - 1) / CB);
    if (grid <= 2L * cus) return R;
  }
  return 16;
}

// mode 0 wkv, 1 delta, 2 mlstm; q / k / v bf16 or fp32 (in_f32) with row strides in elements; rows: rows of the step.
extern "C" int dgi_linear_scan(float* y, int mode, const void* q, int q_stride, const void* k, int k_stride, const void* v,
                               int v_stride, int in_f32, const float* aux1, int aux1_stride, const float* aux2,
                               int aux2_stride, const float* par1, const float* par2, float* state, float* norm, float* mx,
                               const int* positions, const int* seq_row0, const int* seq_slots, int n_seq, int H, int G,
                               int dk, int dv, float cap, int rows, float* norm_new, float* mx_new, hipStream_t st) {
  if (n_seq == 0) return 0;
  if (mode < 0 || mode > 2 || H <= 0 || G <= 0 || H % G || dk <= 0 || dv <= 0) return -2;
  if (dk > 512) return -3;
  if (mode == MLSTM && (!norm || !mx || !aux2 || cap <= 0.f)) return -4;
  if (mode == WKV && (!par1 || !par2)) return -4;
  if (mode == DELTA && (!par1 || !par2 || !aux2)) return -4;
  const bool short_rows = rows <= 4 * n_seq;       // rows of the step: at most four per sequence on average
  const int R = scan_channels(dk, dv, H, n_seq, rows);
  int KS = 1;
  while (KS * R < dk) KS <<= 1;
  if (KS > 16) return -5;
  ScanArgs a;
  a.y = y; a.q = q; a.k = k; a.v = v;
  a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride;
  a.aux1 = aux1; a.aux2 = aux2; a.aux1_stride = aux1_stride; a.aux2_stride = aux2_stride;
  a.par1 = par1; a.par2 = par2; a.state = state; a.norm = norm; a.mx = mx;
  a.positions = positions; a.seq_row0 = seq_row0; a.seq_slots = seq_slots;
  a.H = H; a.G = G; a.dk = dk; a.dv = dv; a.cap = cap;
  a.KS = KS; a.CW = 64 / KS;
  a.CB = scan_columns(KS, dv);
  a.nwc = a.CB / a.CW;
  const int nz = (dv + a.CB - 1) / a.CB;
  if (H > 65535 || nz > 65535) return -5;
  const bool staged = mode == MLSTM && nz > 1;
  if (staged && (!norm_new || !mx_new)) return -7;
  a.norm_new = staged ? norm_new : nullptr;
  a.mx_new = staged ? mx_new : nullptr;
  const dim3 grid(n_seq, H, nz);
  int rc;
#define DGI_SCAN(M_)                                                                                      \
  rc = in_f32 ? launch_scan<M_, float>(a, R, short_rows, grid, st) : launch_scan<M_, uint16_t>(a, R, short_rows, grid, st)
  if (mode == WKV) DGI_SCAN(WKV);
  else if (mode == DELTA) DGI_SCAN(DELTA);
  else DGI_SCAN(MLSTM);
#undef DGI_SCAN
  if (rc) return rc;
  DGI_CHECK_LAUNCH();
  if (staged) {
    mlstm_commit_kernel<<<n_seq, 256, 0, st>>>(norm, mx, norm_new, mx_new, seq_row0, seq_slots, H, dk);
    DGI_CHECK_LAUNCH();
  }
  return 0;
}

// value columns one workgroup covers in this step (the matrix memory stages its normaliser when dv exceeds it)
extern "C" int dgi_linear_scan_columns(int dk, int dv, int H, int n_seq, int rows) {
  const int R = scan_channels(dk, dv, H, n_seq, rows);
  int KS = 1;
  while (KS * R < dk) KS <<= 1;
  if (KS > 16) return 0;
  return scan_columns(KS, dv);
}

extern "C" int dgi_token_shift(void* out, int out_f32, const void* h, int h_f32, int h_stride, const float* mu, int nmix,
                               float* tail, const int* positions, const int* row_seq, const int* seq_row0,
                               const int* seq_slots, int n_seq, int T, int W, hipStream_t st) {
  if (T == 0 || W == 0 || nmix == 0) return 0;
#define DGI_TS(TH_, TO_)                                                                                               \
  token_shift_kernel<TH_, TO_><<<T, 256, 0, st>>>((TO_*)out, (const TH_*)h, h_stride, mu, nmix, tail, positions, row_seq, \
                                                  seq_row0, seq_slots, T, W)
  if (h_f32) { if (out_f32) DGI_TS(float, float); else DGI_TS(float, uint16_t); }
  else { if (out_f32) DGI_TS(uint16_t, float); else DGI_TS(uint16_t, uint16_t); }
#undef DGI_TS
  DGI_CHECK_LAUNCH();
  if (h_f32) token_shift_tail_kernel<float><<<n_seq, 256, 0, st>>>((const float*)h, h_stride, tail, seq_row0, seq_slots, W);
  else token_shift_tail_kernel<uint16_t><<<n_seq, 256, 0, st>>>((const uint16_t*)h, h_stride, tail, seq_row0, seq_slots, W);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_head_norm_gate(void* out, int out_f32, const float* y, const void* z, int z_f32, int z_stride,
                                  const float* w, int wlen, int T, int H, int dv, float eps, int sigmoid_gate,
                                  hipStream_t st) {
  if (T == 0) return 0;
  if (H <= 0 || dv <= 0 || wlen <= 0 || (H * dv) % wlen) return -2;
  const long long units = (long long)T * H;
  // 16-byte path: head sizes, weight period, row strides and pointers in fours
  const bool vec = dv % 4 == 0 && dv <= 256 && wlen % 4 == 0 && z_stride % 4 == 0 &&
                   (((uintptr_t)out | (uintptr_t)y | (uintptr_t)z | (uintptr_t)w) & 15) == 0;
  const unsigned blocks = (unsigned)(vec ? (units + 15) / 16 : (units + 3) / 4);
#define DGI_HNG(TZ_, TO_)                                                                                             \
  do {                                                                                                                \
    if (vec) head_norm_gate_vec_kernel<TZ_, TO_><<<blocks, 256, 0, st>>>((TO_*)out, y, (const TZ_*)z, z_stride, w, wlen, T, H, \
                                                                        dv, eps, sigmoid_gate);                       \
    else head_norm_gate_kernel<TZ_, TO_><<<blocks, 256, 0, st>>>((TO_*)out, y, (const TZ_*)z, z_stride, w, wlen, T, H, dv, eps, \
                                                                sigmoid_gate);                                        \
  } while (0)
  if (z_f32) { if (out_f32) DGI_HNG(float, float); else DGI_HNG(float, uint16_t); }
  else { if (out_f32) DGI_HNG(uint16_t, float); else DGI_HNG(uint16_t, uint16_t); }
#undef DGI_HNG
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_rms_pair_mean(float* out, const void* a, int a_stride, const void* b, int b_stride, int in_f32,
                                 const float* wa, const float* wb, int T, int W, float eps, hipStream_t st) {
  if (T == 0 || W == 0) return 0;
  if (in_f32)
    rms_pair_mean_kernel<float><<<T, 256, 0, st>>>(out, (const float*)a, a_stride, (const float*)b, b_stride, wa, wb, W, eps);
  else
    rms_pair_mean_kernel<uint16_t><<<T, 256, 0, st>>>(out, (const uint16_t*)a, a_stride, (const uint16_t*)b, b_stride, wa,
                                                      wb, W, eps);
  DGI_CHECK_LAUNCH();
  return 0;
}
