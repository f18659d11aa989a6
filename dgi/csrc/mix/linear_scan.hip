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
// linear_scan layout.  A workgroup owns (sequence, head, CB value columns).  Inside a wave, lane = s * CW + j:
// column j of the wave's CW columns, key slice s of KS = 64 / CW slices; a thread keeps R consecutive key
// channels of its column in registers (KS * R >= dk), so a token costs R fused multiply-adds per pass and the
// sums over the key dimension finish with log2(KS) shuffles inside the wave — no barrier per token.
// Tokens are staged TT at a time: every thread loads one key channel (and one value column) of each token into
// registers while the previous tile is computed, the tile then goes to LDS (slices padded apart so the KS
// broadcast reads of a wave hit different banks), per-token scalars (unit norms, decays, gates, the bonus dot
// product, the stabiliser's running maximum) are computed once per token by one wave or one thread, and the
// token loop reads LDS only.  Everything is fp32; q / k / v arrive as bf16 or fp32.
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

__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float logsigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

template <int MODE, typename TI, int R>
__global__ __launch_bounds__(512) void linear_scan_kernel(const ScanArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int seq = blockIdx.x, head = blockIdx.y, cblk = blockIdx.z;
  const int row0 = a.seq_row0[seq], n = a.seq_row0[seq + 1] - row0;
  if (n <= 0) return;
  const int p0 = a.positions[row0], slot = a.seq_slots[seq];
  const int dk = a.dk, dv = a.dv, H = a.H;
  const int kvh = head / (H / a.G);
  const int KS = a.KS, CW = a.CW, CB = a.CB;
  const int KP = KS * (R + 4);                     // padded key row in LDS
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int s = lane / CW, jl = lane - s * CW;
  const bool computes = wave < a.nwc;
  const int cl = wave * CW + jl;                   // column inside the workgroup
  const int col = cblk * CB + cl;
  const bool col_ok = computes && col < dv;
  constexpr int NV = MODE == WKV ? 3 : 2;
  float* sk = sm;                                  // [TT][KP]
  float* sq = sk + TT * KP;
  float* sw = sq + TT * KP;                        // wkv only
  float* sv = sm + NV * TT * KP;                   // [TT][CB]
  float* sc = sv + TT * CB;                        // [TT][4]

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

  // this thread's staged elements: key channel tid of every token, value column cblk * CB + tid
  const bool ld_k = tid < dk, ld_pad = tid < KS * R, ld_v = tid < CB;
  const bool v_ok = ld_v && cblk * CB + tid < dv;
  const int kpi = (tid / R) * (R + 4) + (tid % R);
  const TI* qp = (const TI*)a.q + (size_t)kvh * dk + tid;
  const TI* kp = (const TI*)a.k + (size_t)kvh * dk + tid;
  const TI* vp = (const TI*)a.v + (size_t)head * dv + cblk * CB + tid;
  float w0 = 0.f;
  if (MODE == WKV && ld_k) w0 = a.par1[head * dk + tid];
  float pk[TT], pq[TT], pw[MODE == WKV ? TT : 1], pv[TT];
  auto load_tile = [&](int t0) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      const bool ok = t0 + tt < n;
      const size_t row = (size_t)(row0 + t0 + tt);
      pk[tt] = (ok && ld_k) ? ldf<TI>(kp + row * a.k_stride) : 0.f;
      pq[tt] = (ok && ld_k) ? ldf<TI>(qp + row * a.q_stride) : 0.f;
      if constexpr (MODE == WKV) pw[tt] = (ok && ld_k) ? expf(-expf(a.aux1[row * a.aux1_stride + head * dk + tid] + w0)) : 0.f;
      pv[tt] = (ok && v_ok) ? ldf<TI>(vp + row * a.v_stride) : 0.f;
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      if (ld_pad) {
        sk[tt * KP + kpi] = pk[tt];
        sq[tt * KP + kpi] = pq[tt];
        if constexpr (MODE == WKV) sw[tt * KP + kpi] = pw[tt];
      }
      if (ld_v) sv[tt * CB + tid] = pv[tt];
    }
  };
  const int nwaves = blockDim.x >> 6;
  const float qscale = 1.f / sqrtf((float)dk);

  load_tile(0);
  for (int t0 = 0; t0 < n; t0 += TT) {
    const int nt = min(TT, n - t0);
    store_tile();
    __syncthreads();
    // ---- per-token scalars
    if (MODE == MLSTM) {
      if (tid == 0) {
        for (int tt = 0; tt < nt; ++tt) {
          const size_t row = (size_t)(row0 + t0 + tt);
          const float ig = a.cap * tanhf(a.aux1[row * a.aux1_stride + head] / a.cap);
          const float fg = logsigmoid_f(a.cap * tanhf(a.aux2[row * a.aux2_stride + head] / a.cap));
          const float m_new = fmaxf(fg + m_run, ig);
          sc[tt * 4 + 0] = expf(fg + m_run - m_new);
          sc[tt * 4 + 1] = expf(ig - m_new);
          sc[tt * 4 + 2] = expf(-m_new);
          m_run = m_new;
        }
      }
    } else {
      for (int tt = wave; tt < nt; tt += nwaves) {
        float r1 = 0.f, r2 = 0.f;
        for (int i = lane; i < dk; i += 64) {
          const int pi = (i / R) * (R + 4) + (i % R);
          const float kv = sk[tt * KP + pi], qv = sq[tt * KP + pi];
          if (MODE == WKV) {
            r1 += qv * kv * a.par2[head * dk + i];            // the bonus: sum_i r_i u_i k_i
          } else {
            r1 += kv * kv;
            r2 += qv * qv;
          }
        }
        r1 = wave_sum(r1);
        if (MODE == DELTA) r2 = wave_sum(r2);
        if (lane == 0) {
          if (MODE == WKV) {
            sc[tt * 4] = r1;
          } else {
            const size_t row = (size_t)(row0 + t0 + tt);
            const float dt = softplus_f(a.aux2[row * a.aux2_stride + head] + a.par2[head]);
            sc[tt * 4 + 0] = expf(-expf(a.par1[head]) * dt);                        // decay
            sc[tt * 4 + 1] = 1.f / (1.f + expf(-a.aux1[row * a.aux1_stride + head]));   // write strength
            sc[tt * 4 + 2] = 1.f / sqrtf(r1 + 1e-6f);                               // 1 / |k|
            sc[tt * 4 + 3] = qscale / sqrtf(r2 + 1e-6f);                            // dk^-1/2 / |q|
          }
        }
      }
    }
    __syncthreads();
    if (t0 + TT < n) load_tile(t0 + TT);             // in flight while this tile is computed
    if (computes) {
      for (int tt = 0; tt < nt; ++tt) {
        const float* kk = sk + tt * KP + s * (R + 4);
        const float* qq = sq + tt * KP + s * (R + 4);
        const float vj = sv[tt * CB + cl];
        float o;
        if constexpr (MODE == WKV) {
          const float* ww = sw + tt * KP + s * (R + 4);
          float acc = 0.f;
#pragma unroll
          for (int i = 0; i < R; ++i) acc += S[i] * qq[i];
#pragma unroll
          for (int i = 0; i < R; ++i) S[i] = ww[i] * S[i] + kk[i] * vj;
          for (int off = CW; off < 64; off <<= 1) acc += __shfl_xor(acc, off, 64);
          o = acc + sc[tt * 4] * vj;
        } else if constexpr (MODE == DELTA) {
          const float g = sc[tt * 4], beta = sc[tt * 4 + 1], rk = sc[tt * 4 + 2], rq = sc[tt * 4 + 3];
          float pred = 0.f;
#pragma unroll
          for (int i = 0; i < R; ++i) pred += S[i] * kk[i];
          for (int off = CW; off < 64; off <<= 1) pred += __shfl_xor(pred, off, 64);
          const float ku = beta * (vj - pred * g * rk) * rk;
          float acc = 0.f;
#pragma unroll
          for (int i = 0; i < R; ++i) {
            S[i] = g * S[i] + kk[i] * ku;
            acc += S[i] * qq[i];
          }
          for (int off = CW; off < 64; off <<= 1) acc += __shfl_xor(acc, off, 64);
          o = acc * rq;
        } else {
          const float fa = sc[tt * 4], fb = sc[tt * 4 + 1], em = sc[tt * 4 + 2];
          const float bv = fb * vj;
          float acc = 0.f, nq = 0.f;
#pragma unroll
          for (int i = 0; i < R; ++i) {
            S[i] = fa * S[i] + kk[i] * bv;
            acc += S[i] * qq[i];
            N[i] = fa * N[i] + fb * kk[i];
            nq += N[i] * qq[i];
          }
          for (int off = CW; off < 64; off <<= 1) {
            acc += __shfl_xor(acc, off, 64);
            nq += __shfl_xor(nq, off, 64);
          }
          o = acc * qscale / (fmaxf(fabsf(nq * qscale), em) + 1e-6f);
        }
        if (s == 0 && col_ok) a.y[(size_t)(row0 + t0 + tt) * H * dv + (size_t)head * dv + col] = o;
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

template <int MODE, typename TI>
int launch_scan(const ScanArgs& a, int R, int n_seq, int nthreads, dim3 grid, hipStream_t st) {
  const int NV = MODE == WKV ? 3 : 2;
  const size_t lds = (size_t)(NV * TT * a.KS * (R + 4) + TT * a.CB + TT * 4) * sizeof(float);
  if (lds > 64 * 1024) return -6;
  if (R == 16) linear_scan_kernel<MODE, TI, 16><<<grid, nthreads, lds, st>>>(a);
  else if (R == 32) linear_scan_kernel<MODE, TI, 32><<<grid, nthreads, lds, st>>>(a);
  else linear_scan_kernel<MODE, TI, 64><<<grid, nthreads, lds, st>>>(a);
  return 0;
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

// mode 0 wkv, 1 delta, 2 mlstm; q / k / v bf16 or fp32 (in_f32) with row strides in elements.
// r_sel > 0 forces the key channels per thread (16 / 32 / 64), 0 picks them from dk.
extern "C" int dgi_linear_scan(float* y, int mode, const void* q, int q_stride, const void* k, int k_stride, const void* v,
                               int v_stride, int in_f32, const float* aux1, int aux1_stride, const float* aux2,
                               int aux2_stride, const float* par1, const float* par2, float* state, float* norm, float* mx,
                               const int* positions, const int* seq_row0, const int* seq_slots, int n_seq, int H, int G,
                               int dk, int dv, float cap, int r_sel, float* norm_new, float* mx_new, hipStream_t st) {
  if (n_seq == 0) return 0;
  if (mode < 0 || mode > 2 || H <= 0 || G <= 0 || H % G || dk <= 0 || dv <= 0) return -2;
  if (dk > 512) return -3;
  if (mode == MLSTM && (!norm || !mx || !aux2 || cap <= 0.f)) return -4;
  if (mode == WKV && (!par1 || !par2)) return -4;
  if (mode == DELTA && (!par1 || !par2 || !aux2)) return -4;
  int R = r_sel > 0 ? r_sel : (dk <= 256 ? 16 : 32);
  if (R != 16 && R != 32 && R != 64) return -5;
  int KS = 1;
  while (KS * R < dk) KS <<= 1;
  if (KS > 64) return -5;
  ScanArgs a;
  a.y = y; a.q = q; a.k = k; a.v = v;
  a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride;
  a.aux1 = aux1; a.aux2 = aux2; a.aux1_stride = aux1_stride; a.aux2_stride = aux2_stride;
  a.par1 = par1; a.par2 = par2; a.state = state; a.norm = norm; a.mx = mx;
  a.positions = positions; a.seq_row0 = seq_row0; a.seq_slots = seq_slots;
  a.H = H; a.G = G; a.dk = dk; a.dv = dv; a.cap = cap;
  a.KS = KS; a.CW = 64 / KS;
  a.nwc = (dv + a.CW - 1) / a.CW;
  if (a.nwc > 4) a.nwc = 4;
  a.CB = a.nwc * a.CW;
  const int lw = (KS * R + 63) / 64;
  const int nthreads = 64 * (a.nwc > lw ? a.nwc : lw);
  if (nthreads > 512) return -5;
  const int nz = (dv + a.CB - 1) / a.CB;
  if (H > 65535 || nz > 65535) return -5;
  const bool staged = mode == MLSTM && nz > 1;
  if (staged && (!norm_new || !mx_new)) return -7;
  a.norm_new = staged ? norm_new : nullptr;
  a.mx_new = staged ? mx_new : nullptr;
  const dim3 grid(n_seq, H, nz);
  int rc;
#define DGI_SCAN(M_)                                                                                      \
  rc = in_f32 ? launch_scan<M_, float>(a, R, n_seq, nthreads, grid, st) : launch_scan<M_, uint16_t>(a, R, n_seq, nthreads, grid, st)
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

// value columns one workgroup covers for this key size (the matrix memory stages its normaliser when dv exceeds it)
extern "C" int dgi_linear_scan_columns(int dk, int dv, int r_sel) {
  int R = r_sel > 0 ? r_sel : (dk <= 256 ? 16 : 32);
  int KS = 1;
  while (KS * R < dk) KS <<= 1;
  if (KS > 64) return 0;
  const int CW = 64 / KS;
  int nwc = (dv + CW - 1) / CW;
  if (nwc > 4) nwc = 4;
  return nwc * CW;
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
  const unsigned blocks = (unsigned)((units + 3) / 4);
#define DGI_HNG(TZ_, TO_)                                                                                             \
  head_norm_gate_kernel<TZ_, TO_><<<blocks, 256, 0, st>>>((TO_*)out, y, (const TZ_*)z, z_stride, w, wlen, T, H, dv, eps, \
                                                          sigmoid_gate)
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
