// dgi/csrc/mix/bindings.cpp — torch.ops.dgi.* entries of the mixer-block kernels (dgi/_C_mix.so):
// Dynamic-Tanh norms, per-head q/k norm + rotary + paged KV write, row-wise masked attention,
// clamped GLU and soft-capped logits.  A library of its own, so a model that needs only these
// builds in seconds; it registers into the same `dgi` namespace as dgi/_C.so (as a fragment).
// Shapes are checked here, on the host, before any launch; every op runs on the current stream
// and allocates nothing (one exception: a matrix-memory scan whose heads span several workgroups
// stages two small rows per sequence, from the caching allocator).
#include <torch/library.h>
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
int dgi_dyt(const float* x, const float* alpha, const float* w, const float* b, void* y, int is_f32, int T, int W,
            hipStream_t s);
int dgi_dyt_add(const void* h, int h_stride, const float* alpha1, const float* w1, const float* b1, const float* ls,
                float* res, const float* alpha2, const float* w2, const float* b2, void* y, int is_f32, int T, int W,
                hipStream_t s);
int dgi_embed_dyt(const long long* ids, const void* table, int vocab, float scale, const float* alpha, const float* w,
                  const float* b, float* res, int is_f32, int T, int W, hipStream_t s);
int dgi_qknorm_rope_cache(void* qkv, int is_f32, int T, int stride, const int* positions, const int* slots,
                          const float* qw, const float* kw, float eps, const float* cos_sin, int rd, int H, int G,
                          int dk, int dv, void* k_cache, void* v_cache, int block_size, float qt_coef, int qt_every,
                          hipStream_t s);
int dgi_masked_attn_rows(const void* q, int q_stride, const void* k_cache, const void* v_cache, const int* block_tables,
                         int bt_stride, const int* cu_seqlens, int n_seqs, const int* positions, int rows, int H, int G,
                         int dk, int dv, int block_size, float scale, int mask, const void* gate, int gate_stride,
                         void* out, int out_stride, int is_f32, const float* dist_bias, int n_dist, float softcap,
                         const float* sinks, hipStream_t s);
int dgi_paged_prefill_masked(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                             const int* block_tables, int bt_stride, const int* cu_seqlens_q, const int* context_lens,
                             const int* tiles, int n_tiles, void* out, int out_stride, int nh, int nkv, int hd,
                             int block_size, float scale, int mask, const void* gate, int gate_stride,
                             const float* dist_bias, int n_dist, float softcap, const float* sinks, hipStream_t s);
int dgi_glu_clamped(const void* gu, int gu_stride, void* out, int is_f32, int T, int I, float limit, float alpha,
                    hipStream_t s);
int dgi_scale_softcap(const void* x, int x_stride, float* out, int is_f32, int T, int V, float scale, float cap,
                      hipStream_t s);
int dgi_embed_streams(float* xs, int S, int T, int W, const int* ids, const int* positions, const int* row_seq,
                      const int* seq_row0, const int* seq_slots, int n_seq, int* prev_tok, const void* embed, int vocab,
                      const void* bigram, int buckets, long long mul_prev, long long mul_cur, const void* pos_table,
                      int max_pos, int is_f32, hipStream_t s);
int dgi_hc_mix_norm(float* xs, int S, int T, int W, const void* y, int y_stride, const void* gate, int gate_stride,
                    const float* gate_b, const float* mixm, const float* outc, const float* in_next, const float* norm_w,
                    float eps, float* h32, void* hd, int is_f32, hipStream_t s);
int dgi_causal_conv(void* out, int out_f32, const void* x, int x_f32, int x_stride, int T, int C, int taps, const float* w,
                    const float* bias, float* tail, const int* positions, const int* row_seq, const int* seq_row0,
                    const int* seq_slots, int n_seq, int act, int residual, hipStream_t s);
int dgi_ssm_scan(float* y, const float* xbc, int xbc_stride, const void* dt_raw, int dt_f32, int dt_stride,
                 const float* dt_bias, const float* a_log, const float* d_skip, float* state, const int* positions,
                 const int* seq_row0, const int* seq_slots, int n_seq, int heads, int dv, int N, int G, float* ws,
                 float* wsd, int L, int nchunks, hipStream_t s);
int dgi_gated_group_norm(void* out, int out_f32, const float* y, const void* z, int z_f32, int z_stride, const float* w,
                         int T, int C, int groups, float eps, hipStream_t s);
int dgi_moe_route(int* idx, float* wts, const float* logits, int l_stride, const float* corr, int T, int R, int top,
                  int sigmoid, hipStream_t s);
int dgi_glu_rows(void* out, const void* gu, int gu_stride, int rows, int I, int kind, float limit, float alpha,
                 const float* row_scale, int is_f32, hipStream_t s);
int dgi_stream_add_norm(float* x, int T, int W, const void* y, int y_stride, int y_f32, const float* post_w,
                        const float* next_w, float eps, void* out, int out_f32, const void* y2, int y2_stride, int y2_f32,
                        hipStream_t s);
int dgi_linear_scan(float* y, int mode, const void* q, int q_stride, const void* k, int k_stride, const void* v,
                    int v_stride, int in_f32, const float* aux1, int aux1_stride, const float* aux2, int aux2_stride,
                    const float* par1, const float* par2, float* state, float* norm, float* mx, const int* positions,
                    const int* seq_row0, const int* seq_slots, int n_seq, int H, int G, int dk, int dv, float cap,
                    int rows, float* norm_new, float* mx_new, hipStream_t st);
int dgi_linear_scan_columns(int dk, int dv, int H, int n_seq, int rows);
int dgi_token_shift(void* out, int out_f32, const void* h, int h_f32, int h_stride, const float* mu, int nmix, float* tail,
                    const int* positions, const int* row_seq, const int* seq_row0, const int* seq_slots, int n_seq, int T,
                    int W, hipStream_t st);
int dgi_head_norm_gate(void* out, int out_f32, const float* y, const void* z, int z_f32, int z_stride, const float* w,
                       int wlen, int T, int H, int dv, float eps, int sigmoid_gate, hipStream_t st);
int dgi_rms_pair_mean(float* out, const void* a, int a_stride, const void* b, int b_stride, int in_f32, const float* wa,
                      const float* wb, int T, int W, float eps, hipStream_t st);
int dgi_qk_prep(void* qkv, int is_f32, int T, int stride, const int* positions, const int* slots, const float* qw,
                const float* kw, float eps, const float* cos_sin, int rd, int H, int G, int dk, int dv, void* k_cache,
                void* v_cache, int block_size, int full, int half, hipStream_t s);
int dgi_latent_prep(const void* proj, int stride, int is_f32, int T, int q_rank, int kv_rank, int rot_dim,
                    const float* dq_w, const float* dkv_w, float eps, const int* positions, const int* slots,
                    const float* cos_sin, int dims, int interleaved, void* cq, void* cache, hipStream_t s);
int dgi_rotate_heads(void* x, int stride, int is_f32, int T, const int* positions, const float* cos_sin, int dims,
                     int interleaved, int H, int hs, int off, hipStream_t s);
int dgi_gate_heads(void* out, const void* ov, long long ov_hs, long long ov_ts, const void* gate, int gate_stride,
                   int per_head, int T, int H, int dv, int is_f32, hipStream_t s);
int dgi_gelu_tanh(void* out, const void* x, int x_stride, int rows, int n, const void* table, int t_stride, int vocab,
                  const int* ids, int col0, int is_f32, hipStream_t s);
int dgi_latent_attn_rows(const void* q, int q_stride, const void* q_lat, long long ql_hs, long long ql_ts,
                         const void* cache, const int* block_tables, int bt_stride, const int* cu_seqlens, int n_seqs,
                         const int* positions, int rows, int H, int dim, int rd, int kr, int block_size, float scale,
                         int window, const float* cos_sin, int dims, int interleaved, void* out, long long o_hs,
                         long long o_ts, int is_f32, int nsplit, float* part_o, float* part_ml, int mfma, hipStream_t s);
int dgi_glu_silu(void* out, const void* gu, int gu_stride, int rows, int I, int is_f32, hipStream_t s);
int dgi_moe_expert_gate_up(float* mid, const void* h, int h_stride, const int* idx, const void* gate_up, int T, int E,
                           int top, int ff, int W, const float* pair_scale, int act, float limit, float alpha, int is_f32,
                           hipStream_t s);
int dgi_moe_expert_down(void* ys, const float* mid, const int* idx, const void* down, int T, int E, int top, int ff, int W,
                        int is_f32, hipStream_t s);
int dgi_moe_combine(void* out, const void* ys, const int* where, const void* h, int h_stride, const int* idx,
                    const float* wts, const void* shared, int shared_stride, int T, int E, int top, int W, int is_f32,
                    hipStream_t s);
}

namespace {

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

void check_rc(int rc, const char* what) {
  TORCH_CHECK(rc == 0, "dgi kernel ", what, " failed with code ", rc,
              rc > 0 ? (std::string(" (") + hipGetErrorString((hipError_t)rc) + ")") : std::string());
}

// activation tensors: bf16 or fp32; returns 1 for fp32
int act_kind(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat, name, " must be bfloat16 or float32");
  return t.scalar_type() == at::kFloat ? 1 : 0;
}
void check_f32(const at::Tensor& t, const char* name, int64_t numel = -1) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, " must be a contiguous fp32 GPU tensor");
  TORCH_CHECK(numel < 0 || t.numel() == numel, name, " has ", t.numel(), " elements, expected ", numel);
}
void check_i32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name, " must be a contiguous int32 GPU tensor");
}
void check_rows(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1, name, " must be 2-D with unit column stride");
  TORCH_CHECK(t.size(0) == 0 || t.stride(0) < (int64_t(1) << 31), name, " row stride too large");
}

void dyt(at::Tensor y, const at::Tensor& x, const at::Tensor& alpha, const at::Tensor& w, const at::Tensor& b) {
  const int f = act_kind(y, "y");
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && y.is_contiguous() && y.sizes() == x.sizes());
  const int T = (int)x.size(0), W = (int)x.size(1);
  check_f32(x, "x"); check_f32(alpha, "alpha", 1); check_f32(w, "w", W); check_f32(b, "b", W);
  check_rc(dgi_dyt(x.data_ptr<float>(), alpha.data_ptr<float>(), w.data_ptr<float>(), b.data_ptr<float>(), y.data_ptr(), f,
                   T, W, cur_stream()), "dyt");
}

void dyt_add(at::Tensor res, const at::Tensor& h, const at::Tensor& alpha1, const at::Tensor& w1, const at::Tensor& b1,
             const at::Tensor& ls, const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& alpha2,
             const c10::optional<at::Tensor>& w2, const c10::optional<at::Tensor>& b2) {
  const int f = act_kind(h, "h");
  check_rows(h, "h");
  TORCH_CHECK(res.dim() == 2 && h.size(0) == res.size(0) && h.size(1) == res.size(1));
  const int T = (int)res.size(0), W = (int)res.size(1);
  check_f32(res, "res"); check_f32(alpha1, "alpha1", 1); check_f32(w1, "w1", W); check_f32(b1, "b1", W); check_f32(ls, "ls", W);
  void* yp = nullptr;
  const float *a2 = nullptr, *w2p = nullptr, *b2p = nullptr;
  if (y.has_value()) {
    TORCH_CHECK(alpha2.has_value() && w2.has_value() && b2.has_value(), "dyt_add: y needs the next norm");
    TORCH_CHECK(act_kind(*y, "y") == f && y->is_contiguous() && y->sizes() == res.sizes());
    check_f32(*alpha2, "alpha2", 1); check_f32(*w2, "w2", W); check_f32(*b2, "b2", W);
    yp = y->data_ptr(); a2 = alpha2->data_ptr<float>(); w2p = w2->data_ptr<float>(); b2p = b2->data_ptr<float>();
  }
  check_rc(dgi_dyt_add(h.data_ptr(), (int)h.stride(0), alpha1.data_ptr<float>(), w1.data_ptr<float>(), b1.data_ptr<float>(),
                       ls.data_ptr<float>(), res.data_ptr<float>(), a2, w2p, b2p, yp, f, T, W, cur_stream()), "dyt_add");
}

void embed_dyt(at::Tensor res, const at::Tensor& ids, const at::Tensor& table, double scale, const at::Tensor& alpha,
               const at::Tensor& w, const at::Tensor& b) {
  const int f = act_kind(table, "table");
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kLong && ids.is_contiguous(), "ids must be contiguous int64");
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous() && res.dim() == 2);
  const int T = (int)ids.numel(), W = (int)table.size(1);
  TORCH_CHECK(res.size(0) == T && res.size(1) == W);
  check_f32(res, "res"); check_f32(alpha, "alpha", 1); check_f32(w, "w", W); check_f32(b, "b", W);
  check_rc(dgi_embed_dyt((const long long*)ids.data_ptr<int64_t>(), table.data_ptr(), (int)table.size(0), (float)scale,
                         alpha.data_ptr<float>(), w.data_ptr<float>(), b.data_ptr<float>(), res.data_ptr<float>(), f, T, W,
                         cur_stream()), "embed_dyt");
}

// qkv rows: [q: H*dk | k: G*dk | v: G*dv | ...]; k_cache [NB, G, bs, dk], v_cache [NB, G, bs, dv]
void qknorm_rope_cache(at::Tensor qkv, const at::Tensor& positions, const at::Tensor& slots, const at::Tensor& qw,
                       const at::Tensor& kw, double eps, const c10::optional<at::Tensor>& cos_sin, int64_t H, int64_t G,
                       int64_t dk, int64_t dv, at::Tensor k_cache, at::Tensor v_cache, double qt_coef, int64_t qt_every) {
  const int f = act_kind(qkv, "qkv");
  check_rows(qkv, "qkv");
  check_i32(positions, "positions"); check_i32(slots, "slots");
  check_f32(qw, "qw", dk); check_f32(kw, "kw", dk);
  const int T = (int)qkv.size(0);
  TORCH_CHECK(positions.numel() == T && slots.numel() == T);
  TORCH_CHECK(qkv.size(1) >= (H + G) * dk + G * dv, "qkv rows too short");
  TORCH_CHECK(act_kind(k_cache, "k_cache") == f && act_kind(v_cache, "v_cache") == f);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == dk && v_cache.size(1) == G && v_cache.size(3) == dv &&
              v_cache.size(0) == k_cache.size(0) && v_cache.size(2) == k_cache.size(2), "cache geometry");
  int rd = 0;
  const float* cs = nullptr;
  if (cos_sin.has_value()) {
    check_f32(*cos_sin, "cos_sin");
    TORCH_CHECK(cos_sin->dim() == 2);
    rd = (int)cos_sin->size(1);
    cs = cos_sin->data_ptr<float>();
  }
  check_rc(dgi_qknorm_rope_cache(qkv.data_ptr(), f, T, (int)qkv.stride(0), positions.data_ptr<int>(), slots.data_ptr<int>(),
                                 qw.data_ptr<float>(), kw.data_ptr<float>(), (float)eps, cs, rd, (int)H, (int)G, (int)dk,
                                 (int)dv, k_cache.data_ptr(), v_cache.data_ptr(), (int)k_cache.size(2), (float)qt_coef,
                                 (int)qt_every, cur_stream()),
           "qknorm_rope_cache");
}

// rows of q (stride q.stride(0), H*dk used columns) attend over their sequence's pages;
// cu_seqlens (n_seqs + 1) maps rows to block-table rows, absent: row i <-> block-table row i
void masked_attn_rows(at::Tensor out, const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                      const at::Tensor& block_tables, const c10::optional<at::Tensor>& cu_seqlens,
                      const at::Tensor& positions, int64_t H, int64_t G, double scale, int64_t mask,
                      const c10::optional<at::Tensor>& gate, const c10::optional<at::Tensor>& dist_bias, double softcap,
                      const c10::optional<at::Tensor>& sinks) {
  const int f = act_kind(q, "q");
  check_rows(q, "q"); check_rows(out, "out");
  TORCH_CHECK(act_kind(out, "out") == f && act_kind(k_cache, "k_cache") == f && act_kind(v_cache, "v_cache") == f);
  const float* sk = nullptr;
  if (sinks.has_value()) {
    check_f32(*sinks, "sinks", H);
    sk = sinks->data_ptr<float>();
  }
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  check_i32(block_tables, "block_tables"); check_i32(positions, "positions");
  TORCH_CHECK(block_tables.dim() == 2);
  const int rows = (int)q.size(0);
  const int dk = (int)k_cache.size(3), dv = (int)v_cache.size(3);
  TORCH_CHECK(k_cache.size(1) == G && v_cache.size(1) == G && v_cache.size(2) == k_cache.size(2));
  TORCH_CHECK(q.size(1) >= H * dk && out.size(0) == rows && out.size(1) >= H * dv && positions.numel() == rows);
  int n_seqs = (int)block_tables.size(0);
  const int* cu = nullptr;
  if (cu_seqlens.has_value()) {
    check_i32(*cu_seqlens, "cu_seqlens");
    TORCH_CHECK(cu_seqlens->numel() == n_seqs + 1);
    cu = cu_seqlens->data_ptr<int>();
  } else {
    TORCH_CHECK(n_seqs >= rows, "one block-table row per query row");
  }
  const void* gp = nullptr;
  int gs = 0;
  if (gate.has_value()) {
    check_rows(*gate, "gate");
    TORCH_CHECK(act_kind(*gate, "gate") == f && gate->size(0) == rows && gate->size(1) >= H * dv);
    gp = gate->data_ptr();
    gs = (int)gate->stride(0);
  }
  const float* db = nullptr;
  int nd = 0;
  if (dist_bias.has_value()) {
    check_f32(*dist_bias, "dist_bias");
    TORCH_CHECK(dist_bias->dim() == 2 && dist_bias->size(1) == H && dist_bias->size(0) >= 1, "dist_bias must be [n, H]");
    db = dist_bias->data_ptr<float>();
    nd = (int)dist_bias->size(0);
  }
  check_rc(dgi_masked_attn_rows(q.data_ptr(), (int)q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                block_tables.data_ptr<int>(), (int)block_tables.stride(0), cu, n_seqs,
                                positions.data_ptr<int>(), rows, (int)H, (int)G, dk, dv, (int)k_cache.size(2), (float)scale,
                                (int)mask, gp, gs, out.data_ptr(), (int)out.stride(0), f, db, nd, (float)softcap, sk,
                                cur_stream()),
           "masked_attn_rows");
}

// bf16, key size == value size in {64, 128}: packed prompt portions (cu_seqlens_q) over
// [cached prefix | new keys]; tiles [n, 2] = (sequence, first row of a 128-row tile)
void paged_prefill_masked(at::Tensor out, const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                          const at::Tensor& block_tables, const at::Tensor& cu_seqlens_q, const at::Tensor& context_lens,
                          const at::Tensor& tiles, int64_t nh, int64_t nkv, double scale, int64_t mask,
                          const c10::optional<at::Tensor>& gate, const c10::optional<at::Tensor>& dist_bias, double softcap,
                          const c10::optional<at::Tensor>& sinks) {
  const float* sk = nullptr;
  if (sinks.has_value()) {
    check_f32(*sinks, "sinks", nh);
    sk = sinks->data_ptr<float>();
  }
  TORCH_CHECK(act_kind(q, "q") == 0 && act_kind(out, "out") == 0 && act_kind(k_cache, "k_cache") == 0 &&
              act_kind(v_cache, "v_cache") == 0, "paged_prefill_masked: bfloat16 only");
  check_rows(q, "q"); check_rows(out, "out");
  check_i32(block_tables, "block_tables"); check_i32(cu_seqlens_q, "cu_seqlens_q");
  check_i32(context_lens, "context_lens"); check_i32(tiles, "tiles");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 && k_cache.sizes() == v_cache.sizes());
  const int hd = (int)k_cache.size(3);
  TORCH_CHECK(k_cache.size(1) == nkv && q.size(1) >= nh * hd && out.size(1) >= nh * hd && out.size(0) == q.size(0));
  TORCH_CHECK(q.stride(0) % 8 == 0 && out.stride(0) % 4 == 0 && q.data_ptr<at::BFloat16>() != nullptr);
  TORCH_CHECK(reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0 && reinterpret_cast<uintptr_t>(out.data_ptr()) % 8 == 0,
              "paged_prefill_masked: q must be 16-byte and out 8-byte aligned");
  const int nb = (int)cu_seqlens_q.numel() - 1;
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(0) >= nb && context_lens.numel() >= nb);
  TORCH_CHECK(tiles.dim() == 2 && tiles.size(1) == 2);
  const void* gp = nullptr;
  int gs = 0;
  if (gate.has_value()) {
    check_rows(*gate, "gate");
    TORCH_CHECK(act_kind(*gate, "gate") == 0 && gate->size(0) == q.size(0) && gate->size(1) >= nh * hd);
    TORCH_CHECK(gate->stride(0) % 4 == 0 && reinterpret_cast<uintptr_t>(gate->data_ptr()) % 8 == 0, "gate alignment");
    gp = gate->data_ptr();
    gs = (int)gate->stride(0);
  }
  const float* dbp = nullptr;
  int ndist = 0;
  if (dist_bias.has_value()) {
    check_f32(*dist_bias, "dist_bias");
    TORCH_CHECK(dist_bias->dim() == 2 && dist_bias->size(1) == nh && dist_bias->size(0) >= 1, "dist_bias must be [n, nh]");
    dbp = dist_bias->data_ptr<float>();
    ndist = (int)dist_bias->size(0);
  }
  check_rc(dgi_paged_prefill_masked(q.data_ptr(), (int)q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                    block_tables.data_ptr<int>(), (int)block_tables.stride(0), cu_seqlens_q.data_ptr<int>(),
                                    context_lens.data_ptr<int>(), tiles.data_ptr<int>(), (int)tiles.size(0), out.data_ptr(),
                                    (int)out.stride(0), (int)nh, (int)nkv, hd, (int)k_cache.size(2), (float)scale, (int)mask,
                                    gp, gs, dbp, ndist, (float)softcap, sk, cur_stream()), "paged_prefill_masked");
}

void glu_clamped(at::Tensor out, const at::Tensor& gu, double limit, double alpha) {
  const int f = act_kind(gu, "gu");
  check_rows(gu, "gu");
  TORCH_CHECK(act_kind(out, "out") == f && out.is_contiguous() && out.dim() == 2 && out.size(0) == gu.size(0) &&
              2 * out.size(1) == gu.size(1));
  check_rc(dgi_glu_clamped(gu.data_ptr(), (int)gu.stride(0), out.data_ptr(), f, (int)gu.size(0), (int)out.size(1),
                           (float)limit, (float)alpha, cur_stream()), "glu_clamped");
}

void scale_softcap(at::Tensor out, const at::Tensor& x, double scale, double cap) {
  const int f = act_kind(x, "x");
  check_rows(x, "x");
  check_f32(out, "out", x.numel());
  check_rc(dgi_scale_softcap(x.data_ptr(), (int)x.stride(0), out.data_ptr<float>(), f, (int)x.size(0), (int)x.size(1),
                             (float)scale, (float)cap, cur_stream()), "scale_softcap");
}

const int* i32p(const at::Tensor& t, const char* name, int64_t numel = -1) {
  check_i32(t, name);
  TORCH_CHECK(numel < 0 || t.numel() == numel, name, " has ", t.numel(), " elements, expected ", numel);
  return t.data_ptr<int>();
}
const float* f32p(const c10::optional<at::Tensor>& t, const char* name, int64_t numel) {
  if (!t.has_value()) return nullptr;
  check_f32(*t, name, numel);
  return t->data_ptr<float>();
}

// xs [S, T, W] fp32 <- embed[id] + bigram[hash(prev, id)] + pos_table[pos]; prev_tok [slots] int32 state
void embed_streams(at::Tensor xs, const at::Tensor& ids, const at::Tensor& positions, const at::Tensor& row_seq,
                   const at::Tensor& seq_row0, const at::Tensor& seq_slots, at::Tensor prev_tok, const at::Tensor& embed,
                   const c10::optional<at::Tensor>& bigram, const c10::optional<at::Tensor>& pos_table, int64_t buckets,
                   int64_t mul_prev, int64_t mul_cur) {
  const int f = act_kind(embed, "embed");
  check_f32(xs, "xs");
  TORCH_CHECK(xs.dim() == 3 && embed.dim() == 2 && embed.is_contiguous());
  const int S = (int)xs.size(0), T = (int)xs.size(1), W = (int)xs.size(2);
  TORCH_CHECK(embed.size(1) == W);
  const int n_seq = (int)seq_slots.numel();
  check_i32(prev_tok, "prev_tok");
  const void *bp = nullptr, *pp = nullptr;
  int max_pos = 0;
  if (bigram.has_value()) {
    TORCH_CHECK(act_kind(*bigram, "bigram") == f && bigram->is_contiguous() && bigram->dim() == 2 && bigram->size(1) == W &&
                bigram->size(0) == buckets + 1, "bigram must be [buckets + 1, W]");
    bp = bigram->data_ptr();
  }
  if (pos_table.has_value()) {
    TORCH_CHECK(act_kind(*pos_table, "pos_table") == f && pos_table->is_contiguous() && pos_table->dim() == 2 &&
                pos_table->size(1) == W);
    pp = pos_table->data_ptr();
    max_pos = (int)pos_table->size(0);
  }
  check_rc(dgi_embed_streams(xs.data_ptr<float>(), S, T, W, i32p(ids, "ids", T), i32p(positions, "positions", T),
                             i32p(row_seq, "row_seq", T), i32p(seq_row0, "seq_row0", n_seq + 1), i32p(seq_slots, "seq_slots"),
                             n_seq, prev_tok.data_ptr<int>(), embed.data_ptr(), (int)embed.size(0), bp, (int)buckets,
                             (long long)mul_prev, (long long)mul_cur, pp, max_pos, f, cur_stream()), "embed_streams");
}

void hc_mix_norm(at::Tensor xs, const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& gate,
                 const c10::optional<at::Tensor>& gate_b, const c10::optional<at::Tensor>& mixm,
                 const c10::optional<at::Tensor>& outc, const c10::optional<at::Tensor>& in_next,
                 const c10::optional<at::Tensor>& norm_w, double eps, c10::optional<at::Tensor> h32,
                 c10::optional<at::Tensor> hd) {
  check_f32(xs, "xs");
  TORCH_CHECK(xs.dim() == 3);
  const int S = (int)xs.size(0), T = (int)xs.size(1), W = (int)xs.size(2);
  int f = hd.has_value() ? 0 : 1;
  const void *yp = nullptr, *gp = nullptr;
  int ys = 0, gs = 0;
  if (y.has_value()) {
    f = act_kind(*y, "y");
    check_rows(*y, "y");
    TORCH_CHECK(y->size(0) == T && y->size(1) == W && mixm.has_value() && outc.has_value(), "hc_mix_norm: y needs mix / out");
    yp = y->data_ptr(); ys = (int)y->stride(0);
    if (gate.has_value()) {
      check_rows(*gate, "gate");
      TORCH_CHECK(act_kind(*gate, "gate") == f && gate->size(0) == T && gate->size(1) == W && gate_b.has_value());
      gp = gate->data_ptr(); gs = (int)gate->stride(0);
    }
  }
  float* hp = nullptr;
  void* hdp = nullptr;
  if (in_next.has_value()) {
    TORCH_CHECK(norm_w.has_value() && h32.has_value(), "hc_mix_norm: the read-out needs norm_w and h32");
    check_f32(*h32, "h32", (int64_t)T * W);
    hp = h32->data_ptr<float>();
    if (hd.has_value()) {
      TORCH_CHECK(f == 0 && hd->scalar_type() == at::kBFloat16 && hd->is_contiguous() && hd->numel() == (int64_t)T * W && hd->is_cuda(),
                  "hc_mix_norm: hd is the bfloat16 copy of h for bfloat16 models");
      hdp = hd->data_ptr();
    }
  }
  check_rc(dgi_hc_mix_norm(xs.data_ptr<float>(), S, T, W, yp, ys, gp, gs, gp ? f32p(gate_b, "gate_b", W) : nullptr,
                           yp ? f32p(mixm, "mix", (int64_t)S * S) : nullptr, yp ? f32p(outc, "out", S) : nullptr,
                           f32p(in_next, "in_next", S), in_next.has_value() ? f32p(norm_w, "norm_w", W) : nullptr,
                           (float)eps, hp, hdp, f, cur_stream()), "hc_mix_norm");
}

void causal_conv(at::Tensor out, const at::Tensor& x, const at::Tensor& w, const c10::optional<at::Tensor>& bias,
                 const c10::optional<at::Tensor>& tail, const at::Tensor& positions, const at::Tensor& row_seq,
                 const at::Tensor& seq_row0, const at::Tensor& seq_slots, int64_t act, bool residual) {
  const int xf = act_kind(x, "x"), of = act_kind(out, "out");
  check_rows(x, "x");
  const int T = (int)x.size(0), C = (int)x.size(1);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == C);
  check_f32(w, "w");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C, "w must be [C, taps]");
  const int taps = (int)w.size(1);
  const int n_seq = (int)seq_slots.numel();
  float* tp = nullptr;
  if (tail.has_value()) {
    check_f32(*tail, "tail");
    TORCH_CHECK(tail->dim() == 3 && tail->size(1) == taps - 1 && tail->size(2) == C, "tail must be [slots, taps - 1, C]");
    tp = tail->data_ptr<float>();
  }
  check_rc(dgi_causal_conv(out.data_ptr(), of, x.data_ptr(), xf, (int)x.stride(0), T, C, taps, w.data_ptr<float>(),
                           f32p(bias, "bias", C), tp, i32p(positions, "positions", T), i32p(row_seq, "row_seq", T),
                           i32p(seq_row0, "seq_row0", n_seq + 1), i32p(seq_slots, "seq_slots"), n_seq, (int)act,
                           residual ? 1 : 0, cur_stream()), "causal_conv");
}

void ssm_scan(at::Tensor y, const at::Tensor& xbc, const at::Tensor& dt_raw, const at::Tensor& dt_bias,
              const at::Tensor& a_log, const at::Tensor& d_skip, at::Tensor state, const at::Tensor& positions,
              const at::Tensor& seq_row0, const at::Tensor& seq_slots, int64_t heads, int64_t dv, int64_t N, int64_t G,
              c10::optional<at::Tensor> ws, c10::optional<at::Tensor> wsd, int64_t L, int64_t nchunks) {
  check_f32(y, "y"); check_f32(xbc, "xbc"); check_f32(state, "state");
  const int df = act_kind(dt_raw, "dt_raw");
  check_rows(dt_raw, "dt_raw");
  const int T = (int)xbc.size(0);
  TORCH_CHECK(xbc.dim() == 2 && xbc.size(1) == heads * dv + 2 * G * N, "xbc must be [T, heads*dv + 2*G*N]");
  TORCH_CHECK(y.numel() == (int64_t)T * heads * dv && dt_raw.size(0) == T && dt_raw.size(1) == heads);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == dv && state.size(3) == N, "state must be [slots, heads, dv, N]");
  check_f32(dt_bias, "dt_bias", heads); check_f32(a_log, "a_log", heads); check_f32(d_skip, "d_skip", heads);
  const int n_seq = (int)seq_slots.numel();
  float *wsp = nullptr, *wdp = nullptr;
  if (ws.has_value()) {
    TORCH_CHECK(wsd.has_value() && L >= 1 && nchunks >= 1, "ssm_scan: the chunked form needs both workspaces");
    check_f32(*ws, "ws", (int64_t)n_seq * nchunks * heads * dv * N);
    check_f32(*wsd, "wsd", (int64_t)n_seq * nchunks * heads);
    TORCH_CHECK(nchunks * L >= T, "ssm_scan: nchunks * L must cover the longest portion");
    wsp = ws->data_ptr<float>(); wdp = wsd->data_ptr<float>();
  }
  check_rc(dgi_ssm_scan(y.data_ptr<float>(), xbc.data_ptr<float>(), (int)xbc.stride(0), dt_raw.data_ptr(), df,
                        (int)dt_raw.stride(0), dt_bias.data_ptr<float>(), a_log.data_ptr<float>(), d_skip.data_ptr<float>(),
                        state.data_ptr<float>(), i32p(positions, "positions", T), i32p(seq_row0, "seq_row0", n_seq + 1),
                        i32p(seq_slots, "seq_slots"), n_seq, (int)heads, (int)dv, (int)N, (int)G, wsp, wdp, (int)L,
                        (int)nchunks, cur_stream()), "ssm_scan");
}

void gated_group_norm(at::Tensor out, const at::Tensor& y, const at::Tensor& z, const at::Tensor& w, int64_t groups,
                      double eps) {
  check_f32(y, "y");
  const int zf = act_kind(z, "z"), of = act_kind(out, "out");
  check_rows(z, "z");
  TORCH_CHECK(y.dim() == 2 && out.is_contiguous() && out.sizes() == y.sizes() && z.size(0) == y.size(0) && z.size(1) == y.size(1));
  check_f32(w, "w", y.size(1));
  check_rc(dgi_gated_group_norm(out.data_ptr(), of, y.data_ptr<float>(), z.data_ptr(), zf, (int)z.stride(0),
                                w.data_ptr<float>(), (int)y.size(0), (int)y.size(1), (int)groups, (float)eps, cur_stream()),
           "gated_group_norm");
}

void moe_route(at::Tensor idx, at::Tensor wts, const at::Tensor& logits, const c10::optional<at::Tensor>& corr,
               int64_t sigmoid) {
  check_i32(idx, "idx"); check_f32(wts, "wts");
  TORCH_CHECK(logits.is_cuda() && logits.scalar_type() == at::kFloat && logits.dim() == 2 && logits.stride(1) == 1);
  const int T = (int)logits.size(0), R = (int)logits.size(1);
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == T && wts.sizes() == idx.sizes());
  check_rc(dgi_moe_route(idx.data_ptr<int>(), wts.data_ptr<float>(), logits.data_ptr<float>(), (int)logits.stride(0),
                         f32p(corr, "correction", R), T, R, (int)idx.size(1), (int)sigmoid, cur_stream()), "moe_route");
}

void glu_silu(at::Tensor out, const at::Tensor& gu) {
  const int f = act_kind(gu, "gu");
  check_rows(gu, "gu");
  TORCH_CHECK(act_kind(out, "out") == f && out.is_contiguous() && out.dim() == 2 && out.size(0) == gu.size(0) &&
              2 * out.size(1) == gu.size(1));
  check_rc(dgi_glu_silu(out.data_ptr(), gu.data_ptr(), (int)gu.stride(0), (int)gu.size(0), (int)out.size(1), f, cur_stream()),
           "glu_silu");
}

// gate_up [E, 2 ff, W], down [E, W, ff] in h's dtype; idx [T, top]; mid [T * top, ff] fp32; ys [T * top, W]
void moe_expert_gate_up(at::Tensor mid, const at::Tensor& h, const at::Tensor& idx, const at::Tensor& gate_up,
                        const c10::optional<at::Tensor>& pair_scale, int64_t act, double limit, double alpha) {
  const int f = act_kind(h, "h");
  check_rows(h, "h"); check_f32(mid, "mid"); check_i32(idx, "idx");
  TORCH_CHECK(act_kind(gate_up, "gate_up") == f && gate_up.is_contiguous() && gate_up.dim() == 3 && gate_up.size(2) == h.size(1));
  const int T = (int)h.size(0), W = (int)h.size(1), E = (int)gate_up.size(0), ff = (int)gate_up.size(1) / 2;
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == T && mid.numel() == (int64_t)T * idx.size(1) * ff);
  check_rc(dgi_moe_expert_gate_up(mid.data_ptr<float>(), h.data_ptr(), (int)h.stride(0), idx.data_ptr<int>(),
                                  gate_up.data_ptr(), T, E, (int)idx.size(1), ff, W, f32p(pair_scale, "pair_scale", idx.numel()),
                                  (int)act, (float)limit, (float)alpha, f, cur_stream()), "moe_expert_gate_up");
}

void moe_expert_down(at::Tensor ys, const at::Tensor& mid, const at::Tensor& idx, const at::Tensor& down) {
  const int f = act_kind(ys, "ys");
  check_f32(mid, "mid"); check_i32(idx, "idx");
  TORCH_CHECK(act_kind(down, "down") == f && down.is_contiguous() && down.dim() == 3);
  const int E = (int)down.size(0), W = (int)down.size(1), ff = (int)down.size(2);
  TORCH_CHECK(idx.dim() == 2 && ys.is_contiguous() && ys.dim() == 2 && ys.size(0) == idx.numel() && ys.size(1) == W &&
              mid.numel() == idx.numel() * ff);
  check_rc(dgi_moe_expert_down(ys.data_ptr(), mid.data_ptr<float>(), idx.data_ptr<int>(), down.data_ptr(), (int)idx.size(0), E,
                               (int)idx.size(1), ff, W, f, cur_stream()), "moe_expert_down");
}

void moe_combine(at::Tensor out, const at::Tensor& ys, const c10::optional<at::Tensor>& where, const at::Tensor& h, const at::Tensor& idx,
                 const c10::optional<at::Tensor>& wts, const c10::optional<at::Tensor>& shared, int64_t E) {
  const int f = act_kind(h, "h");
  check_rows(h, "h"); check_i32(idx, "idx");
  const int* wp = nullptr;
  if (where.has_value()) {
    check_i32(*where, "where");
    TORCH_CHECK(where->numel() == idx.numel());
    wp = where->data_ptr<int>();
  }
  const int T = (int)h.size(0), W = (int)h.size(1);
  TORCH_CHECK(act_kind(out, "out") == f && out.is_contiguous() && out.size(0) == T && out.size(1) == W);
  TORCH_CHECK(act_kind(ys, "ys") == f && ys.is_contiguous() && ys.dim() == 2 && ys.size(1) == W);
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == T);
  TORCH_CHECK(where.has_value() || ys.size(0) == idx.numel(), "moe_combine: without `where` ys holds one row per pair");
  const void* sp = nullptr;
  int ss = 0;
  if (shared.has_value()) {
    check_rows(*shared, "shared");
    TORCH_CHECK(act_kind(*shared, "shared") == f && shared->size(0) == T && shared->size(1) == W);
    sp = shared->data_ptr(); ss = (int)shared->stride(0);
  }
  check_rc(dgi_moe_combine(out.data_ptr(), ys.data_ptr(), wp, h.data_ptr(), (int)h.stride(0),
                           idx.data_ptr<int>(), f32p(wts, "wts", idx.numel()), sp, ss, T, (int)E, (int)idx.size(1), W, f, cur_stream()),
           "moe_combine");
}

void glu_rows(at::Tensor out, const at::Tensor& gu, int64_t kind, double limit, double alpha,
              const c10::optional<at::Tensor>& row_scale) {
  const int f = act_kind(gu, "gu");
  check_rows(gu, "gu");
  TORCH_CHECK(act_kind(out, "out") == f && out.is_contiguous() && out.dim() == 2 && out.size(0) == gu.size(0) &&
              2 * out.size(1) == gu.size(1));
  check_rc(dgi_glu_rows(out.data_ptr(), gu.data_ptr(), (int)gu.stride(0), (int)gu.size(0), (int)out.size(1), (int)kind,
                        (float)limit, (float)alpha, f32p(row_scale, "row_scale", gu.size(0)), f, cur_stream()), "glu_rows");
}

// x [T, W] fp32 += y (unit-RMS normed and weighted if post_w); out = RMS norm of x times next_w (or x) in out's dtype
void stream_add_norm(at::Tensor x, const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& post_w,
                     const c10::optional<at::Tensor>& next_w, double eps, c10::optional<at::Tensor> out,
                     const c10::optional<at::Tensor>& y2) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2);
  const int T = (int)x.size(0), W = (int)x.size(1);
  const void* yp = nullptr;
  int ys = 0, yf = 1;
  if (y.has_value()) {
    yf = act_kind(*y, "y");
    check_rows(*y, "y");
    TORCH_CHECK(y->size(0) == T && y->size(1) == W, "stream_add_norm: y must be [T, W]");
    yp = y->data_ptr(); ys = (int)y->stride(0);
  }
  TORCH_CHECK(!post_w.has_value() || y.has_value(), "stream_add_norm: post_w needs y");
  void* op = nullptr;
  int of = 1;
  if (out.has_value()) {
    of = act_kind(*out, "out");
    TORCH_CHECK(out->is_contiguous() && out->dim() == 2 && out->size(0) == T && out->size(1) == W);
    op = out->data_ptr();
  }
  const void* y2p = nullptr;
  int y2s = 0, y2f = 1;
  if (y2.has_value()) {
    TORCH_CHECK(y.has_value(), "stream_add_norm: y2 needs y");
    y2f = act_kind(*y2, "y2");
    check_rows(*y2, "y2");
    TORCH_CHECK(y2->size(0) == T && y2->size(1) == W, "stream_add_norm: y2 must be [T, W]");
    y2p = y2->data_ptr(); y2s = (int)y2->stride(0);
  }
  check_rc(dgi_stream_add_norm(x.data_ptr<float>(), T, W, yp, ys, yf, f32p(post_w, "post_w", W), f32p(next_w, "next_w", W),
                               (float)eps, op, of, y2p, y2s, y2f, cur_stream()), "stream_add_norm");
}

void latent_prep(at::Tensor cq, const at::Tensor& proj, int64_t q_rank, int64_t kv_rank, int64_t rot_dim,
                 const at::Tensor& dq_w, const c10::optional<at::Tensor>& dkv_w, double eps, const at::Tensor& positions,
                 const at::Tensor& slots, const c10::optional<at::Tensor>& cos_sin, bool interleaved,
                 c10::optional<at::Tensor> cache) {
  const int f = act_kind(proj, "proj");
  check_rows(proj, "proj");
  const int T = (int)proj.size(0);
  TORCH_CHECK(q_rank > 0 && kv_rank >= 0 && rot_dim >= 0 && proj.size(1) >= q_rank + kv_rank + rot_dim,
              "latent_prep: proj rows are [q_rank | kv_rank | rot_dim | ...]");
  TORCH_CHECK(act_kind(cq, "cq") == f && cq.is_contiguous() && cq.dim() == 2 && cq.size(0) == T && cq.size(1) == q_rank);
  check_f32(dq_w, "dq_w", q_rank);
  int dims = 0;
  const float* csp = nullptr;
  void* cp = nullptr;
  if (cache.has_value()) {
    TORCH_CHECK(act_kind(*cache, "cache") == f && cache->is_contiguous() && cache->dim() == 4 && cache->size(1) == 1 &&
                cache->size(3) == kv_rank + rot_dim && kv_rank > 0, "latent_prep: cache must be [NB, 1, bs, kv_rank + rot_dim]");
    TORCH_CHECK(dkv_w.has_value(), "latent_prep: the cached latent needs its norm weight");
    cp = cache->data_ptr();
    if (cos_sin.has_value()) {
      check_f32(*cos_sin, "cos_sin");
      TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) <= rot_dim && cos_sin->size(1) % 2 == 0,
                  "latent_prep: cos_sin must be [max_pos, dims], dims even and at most rot_dim");
      dims = (int)cos_sin->size(1);
      csp = cos_sin->data_ptr<float>();
    }
  }
  check_rc(dgi_latent_prep(proj.data_ptr(), (int)proj.stride(0), f, T, (int)q_rank, (int)kv_rank, (int)rot_dim,
                           dq_w.data_ptr<float>(), cache.has_value() ? f32p(dkv_w, "dkv_w", kv_rank) : nullptr, (float)eps,
                           i32p(positions, "positions", T), i32p(slots, "slots", T), csp, dims, interleaved ? 1 : 0,
                           cq.data_ptr(), cp, cur_stream()), "latent_prep");
}

// [H, T, n] views with unit inner stride: (head stride, row stride)
void check_htn(const at::Tensor& t, const char* name, int64_t H, int64_t T, int64_t n) {
  TORCH_CHECK(t.dim() == 3 && t.size(0) == H && t.size(1) == T && t.size(2) == n && (n == 1 || t.stride(2) == 1), name,
              " must be [H, T, n] with unit inner stride");
}

void latent_attn_rows(at::Tensor out, const at::Tensor& q, const at::Tensor& q_lat, const at::Tensor& cache,
                      const at::Tensor& block_tables, const c10::optional<at::Tensor>& cu_seqlens, const at::Tensor& positions,
                      int64_t H, int64_t dim, int64_t rot_dim, int64_t kv_rank, double scale, int64_t window,
                      const c10::optional<at::Tensor>& cos_sin, bool interleaved, int64_t nsplit,
                      c10::optional<at::Tensor> part_o, c10::optional<at::Tensor> part_ml, bool mfma) {
  const int f = act_kind(q, "q");
  float *pop = nullptr, *pmp = nullptr;
  TORCH_CHECK(nsplit >= 1, "latent_attn_rows: nsplit >= 1");
  const int64_t runs = nsplit;
  if (runs > 1) {
    TORCH_CHECK(part_o.has_value() && part_ml.has_value(), "latent_attn_rows: split runs need their workspaces");
    check_f32(*part_o, "part_o", runs * H * q.size(0) * kv_rank);
    check_f32(*part_ml, "part_ml", runs * H * q.size(0) * 2);
    pop = part_o->data_ptr<float>(); pmp = part_ml->data_ptr<float>();
  }
  check_rows(q, "q");
  const int T = (int)q.size(0);
  TORCH_CHECK(q.size(1) == H * (dim + rot_dim), "latent_attn_rows: q must be [T, H * (dim + rot_dim)]");
  TORCH_CHECK(act_kind(q_lat, "q_lat") == f && act_kind(out, "out") == f && act_kind(cache, "cache") == f);
  check_htn(q_lat, "q_lat", H, T, kv_rank);
  check_htn(out, "out", H, T, kv_rank);
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 4 && cache.size(1) == 1 && cache.size(3) == kv_rank + rot_dim,
              "latent_attn_rows: cache must be [NB, 1, bs, kv_rank + rot_dim]");
  check_i32(block_tables, "block_tables");
  TORCH_CHECK(block_tables.dim() == 2);
  const int* cu = nullptr;
  int n_seqs = (int)block_tables.size(0);
  if (cu_seqlens.has_value()) {
    check_i32(*cu_seqlens, "cu_seqlens");
    n_seqs = (int)cu_seqlens->numel() - 1;
    TORCH_CHECK(n_seqs >= 1 && n_seqs <= block_tables.size(0), "latent_attn_rows: cu_seqlens does not fit the block tables");
    cu = cu_seqlens->data_ptr<int>();
  } else {
    TORCH_CHECK(block_tables.size(0) >= T, "latent_attn_rows: one block-table row per query row");
  }
  int dims = 0;
  const float* csp = nullptr;
  if (cos_sin.has_value()) {
    check_f32(*cos_sin, "cos_sin");
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) <= rot_dim && cos_sin->size(1) % 2 == 0);
    dims = (int)cos_sin->size(1);
    csp = cos_sin->data_ptr<float>();
  }
  check_rc(dgi_latent_attn_rows(q.data_ptr(), (int)q.stride(0), q_lat.data_ptr(), (long long)q_lat.stride(0),
                                (long long)q_lat.stride(1), cache.data_ptr(), block_tables.data_ptr<int>(),
                                (int)block_tables.stride(0), cu, n_seqs, i32p(positions, "positions", T), T, (int)H, (int)dim,
                                (int)rot_dim, (int)kv_rank, (int)cache.size(2), (float)scale, (int)window, csp, dims,
                                interleaved ? 1 : 0, out.data_ptr(), (long long)out.stride(0), (long long)out.stride(1), f,
                                (int)nsplit, pop, pmp, mfma ? 1 : 0, cur_stream()), "latent_attn_rows");
}

void rotate_heads(at::Tensor x, const at::Tensor& positions, const at::Tensor& cos_sin, bool interleaved, int64_t H,
                  int64_t head_size, int64_t offset) {
  const int f = act_kind(x, "x");
  check_rows(x, "x");
  check_f32(cos_sin, "cos_sin");
  TORCH_CHECK(cos_sin.dim() == 2 && x.size(1) >= H * head_size, "rotate_heads: x rows hold H heads of head_size");
  check_rc(dgi_rotate_heads(x.data_ptr(), (int)x.stride(0), f, (int)x.size(0), i32p(positions, "positions", x.size(0)),
                            cos_sin.data_ptr<float>(), (int)cos_sin.size(1), interleaved ? 1 : 0, (int)H, (int)head_size,
                            (int)offset, cur_stream()), "rotate_heads");
}

void gate_heads(at::Tensor out, const at::Tensor& ov, const c10::optional<at::Tensor>& gate, bool per_head) {
  const int f = act_kind(ov, "ov");
  TORCH_CHECK(ov.dim() == 3 && (ov.size(2) == 1 || ov.stride(2) == 1), "gate_heads: ov must be [H, T, dv] with unit inner stride");
  const int H = (int)ov.size(0), T = (int)ov.size(1), dv = (int)ov.size(2);
  TORCH_CHECK(act_kind(out, "out") == f && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == (int64_t)H * dv);
  const void* gp = nullptr;
  int gs = 0;
  if (gate.has_value()) {
    check_rows(*gate, "gate");
    TORCH_CHECK(act_kind(*gate, "gate") == f && gate->size(0) == T && gate->size(1) == (per_head ? H : H * dv),
                "gate_heads: gate must be [T, H] (per head) or [T, H * dv]");
    gp = gate->data_ptr(); gs = (int)gate->stride(0);
  }
  check_rc(dgi_gate_heads(out.data_ptr(), ov.data_ptr(), (long long)ov.stride(0), (long long)ov.stride(1), gp, gs,
                          per_head ? 1 : 0, T, H, dv, f, cur_stream()), "gate_heads");
}

void gelu_tanh(at::Tensor out, const at::Tensor& x, const c10::optional<at::Tensor>& table,
               const c10::optional<at::Tensor>& ids, int64_t col0) {
  const int f = act_kind(x, "x");
  check_rows(x, "x");
  TORCH_CHECK(act_kind(out, "out") == f && out.is_contiguous() && out.sizes() == x.sizes());
  const int T = (int)x.size(0), n = (int)x.size(1);
  const void* tp = nullptr;
  const int* ip = nullptr;
  int ts = 0, vocab = 0;
  if (table.has_value()) {
    check_rows(*table, "table");
    TORCH_CHECK(act_kind(*table, "table") == f && ids.has_value() && col0 >= 0 && col0 + n <= table->size(1),
                "gelu_tanh: table must hold columns [col0, col0 + n) and come with ids");
    tp = table->data_ptr(); ts = (int)table->stride(0); vocab = (int)table->size(0);
    ip = i32p(*ids, "ids", T);
  }
  check_rc(dgi_gelu_tanh(out.data_ptr(), x.data_ptr(), (int)x.stride(0), T, n, tp, ts, vocab, ip, (int)col0, f, cur_stream()),
           "gelu_tanh");
}

// q / k / v: 2-D row views (unit column stride) of bf16 or fp32 activations, all of one dtype; aux1 / aux2 fp32 row views
void linear_scan(at::Tensor y, int64_t mode, const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                 const at::Tensor& aux1, const c10::optional<at::Tensor>& aux2, const c10::optional<at::Tensor>& par1,
                 const c10::optional<at::Tensor>& par2, at::Tensor state, c10::optional<at::Tensor> norm,
                 c10::optional<at::Tensor> mx, const at::Tensor& positions, const at::Tensor& seq_row0,
                 const at::Tensor& seq_slots, int64_t H, int64_t G, int64_t dk, int64_t dv, double cap) {
  check_f32(y, "y"); check_f32(state, "state");
  const int f = act_kind(q, "q");
  TORCH_CHECK(act_kind(k, "k") == f && act_kind(v, "v") == f, "linear_scan: q, k, v must share a dtype");
  check_rows(q, "q"); check_rows(k, "k"); check_rows(v, "v"); check_rows(aux1, "aux1");
  const int T = (int)q.size(0);
  TORCH_CHECK(mode >= 0 && mode <= 2 && H > 0 && G > 0 && H % G == 0);
  TORCH_CHECK(q.size(1) == G * dk && k.size(0) == T && k.size(1) == G * dk && v.size(0) == T && v.size(1) == H * dv,
              "linear_scan: q / k must be [T, G*dk], v [T, H*dv]");
  TORCH_CHECK(y.dim() == 2 && y.size(0) == T && y.size(1) == H * dv);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dk && state.size(3) == dv,
              "state must be [slots, H, dk, dv]");
  TORCH_CHECK(aux1.is_cuda() && aux1.scalar_type() == at::kFloat && aux1.size(0) == T &&
              aux1.size(1) == (mode == 0 ? H * dk : H), "linear_scan: aux1 shape");
  const float* a2 = nullptr;
  int a2s = 0;
  if (aux2.has_value()) {
    check_rows(*aux2, "aux2");
    TORCH_CHECK(aux2->is_cuda() && aux2->scalar_type() == at::kFloat && aux2->size(0) == T && aux2->size(1) == H);
    a2 = aux2->data_ptr<float>(); a2s = (int)aux2->stride(0);
  }
  const int64_t np = mode == 0 ? H * dk : H;
  float *nrm = nullptr, *mxp = nullptr;
  if (mode == 2) {
    TORCH_CHECK(norm.has_value() && mx.has_value(), "linear_scan: the matrix memory needs its normaliser and maximum states");
    check_f32(*norm, "norm"); check_f32(*mx, "mx");
    TORCH_CHECK(norm->dim() == 3 && norm->size(0) == state.size(0) && norm->size(1) == H && norm->size(2) == dk);
    TORCH_CHECK(mx->dim() == 2 && mx->size(0) == state.size(0) && mx->size(1) == H);
    nrm = norm->data_ptr<float>(); mxp = mx->data_ptr<float>();
  }
  const int n_seq = (int)seq_slots.numel();
  // a matrix memory whose heads span several column blocks stages its new normaliser / maximum (committed by a second launch)
  at::Tensor norm_new, mx_new;
  float *nn = nullptr, *mn = nullptr;
  if (mode == 2 && n_seq > 0 && dgi_linear_scan_columns((int)dk, (int)dv, (int)H, n_seq, T) < dv) {
    norm_new = at::empty({n_seq, H, dk}, state.options());
    mx_new = at::empty({n_seq, H}, state.options());
    nn = norm_new.data_ptr<float>(); mn = mx_new.data_ptr<float>();
  }
  check_rc(dgi_linear_scan(y.data_ptr<float>(), (int)mode, q.data_ptr(), (int)q.stride(0), k.data_ptr(), (int)k.stride(0),
                           v.data_ptr(), (int)v.stride(0), f, aux1.data_ptr<float>(), (int)aux1.stride(0), a2, a2s,
                           f32p(par1, "par1", np), f32p(par2, "par2", np), state.data_ptr<float>(), nrm, mxp,
                           i32p(positions, "positions", T), i32p(seq_row0, "seq_row0", n_seq + 1),
                           i32p(seq_slots, "seq_slots"), n_seq, (int)H, (int)G, (int)dk, (int)dv, (float)cap, T,
                           nn, mn, cur_stream()), "linear_scan");
}

// out [n, T, W] <- h + (previous row - h) * mu[n]; tail [slots, W] fp32 holds each sequence's last row
void token_shift(at::Tensor out, const at::Tensor& h, const at::Tensor& mu, at::Tensor tail, const at::Tensor& positions,
                 const at::Tensor& row_seq, const at::Tensor& seq_row0, const at::Tensor& seq_slots) {
  const int hf = act_kind(h, "h"), of = act_kind(out, "out");
  check_rows(h, "h");
  const int T = (int)h.size(0), W = (int)h.size(1);
  check_f32(mu, "mu"); check_f32(tail, "tail");
  TORCH_CHECK(mu.dim() == 2 && mu.size(1) == W && tail.dim() == 2 && tail.size(1) == W);
  const int nmix = (int)mu.size(0);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 3 && out.size(0) == nmix && out.size(1) == T && out.size(2) == W);
  const int n_seq = (int)seq_slots.numel();
  check_rc(dgi_token_shift(out.data_ptr(), of, h.data_ptr(), hf, (int)h.stride(0), mu.data_ptr<float>(), nmix,
                           tail.data_ptr<float>(), i32p(positions, "positions", T), i32p(row_seq, "row_seq", T),
                           i32p(seq_row0, "seq_row0", n_seq + 1), i32p(seq_slots, "seq_slots"), n_seq, T, W, cur_stream()),
           "token_shift");
}

void head_norm_gate(at::Tensor out, const at::Tensor& y, const at::Tensor& z, const at::Tensor& w, int64_t heads, double eps,
                    int64_t sigmoid_gate) {
  check_f32(y, "y"); check_f32(w, "w");
  const int zf = act_kind(z, "z"), of = act_kind(out, "out");
  check_rows(z, "z");
  TORCH_CHECK(y.dim() == 2 && out.is_contiguous() && out.sizes() == y.sizes() && z.size(0) == y.size(0) && z.size(1) == y.size(1));
  const int T = (int)y.size(0), C = (int)y.size(1);
  TORCH_CHECK(heads > 0 && C % heads == 0 && w.numel() > 0 && C % w.numel() == 0, "head_norm_gate: sizes");
  check_rc(dgi_head_norm_gate(out.data_ptr(), of, y.data_ptr<float>(), z.data_ptr(), zf, (int)z.stride(0), w.data_ptr<float>(),
                              (int)w.numel(), T, (int)heads, C / (int)heads, (float)eps, (int)sigmoid_gate, cur_stream()),
           "head_norm_gate");
}

void rms_pair_mean(at::Tensor out, const at::Tensor& a, const at::Tensor& b, const at::Tensor& wa, const at::Tensor& wb,
                   double eps) {
  check_f32(out, "out");
  const int f = act_kind(a, "a");
  TORCH_CHECK(act_kind(b, "b") == f);
  check_rows(a, "a"); check_rows(b, "b");
  const int T = (int)a.size(0), W = (int)a.size(1);
  TORCH_CHECK(b.size(0) == T && b.size(1) == W && out.dim() == 2 && out.size(0) == T && out.size(1) == W);
  check_f32(wa, "wa", W); check_f32(wb, "wb", W);
  check_rc(dgi_rms_pair_mean(out.data_ptr<float>(), a.data_ptr(), (int)a.stride(0), b.data_ptr(), (int)b.stride(0), f,
                             wa.data_ptr<float>(), wb.data_ptr<float>(), T, W, (float)eps, cur_stream()), "rms_pair_mean");
}

// qkv rows: [q: H*dk | k: G*dk | v: G*dv | ...]; full: norm over the whole q / k projection (weights [H*dk] / [G*dk])
void qk_prep(at::Tensor qkv, const at::Tensor& positions, const at::Tensor& slots, const at::Tensor& qw, const at::Tensor& kw,
             double eps, const c10::optional<at::Tensor>& cos_sin, int64_t H, int64_t G, int64_t dk, int64_t dv,
             at::Tensor k_cache, at::Tensor v_cache, bool full, bool half) {
  const int f = act_kind(qkv, "qkv");
  check_rows(qkv, "qkv");
  check_i32(positions, "positions"); check_i32(slots, "slots");
  check_f32(qw, "qw", full ? H * dk : dk); check_f32(kw, "kw", full ? G * dk : dk);
  const int T = (int)qkv.size(0);
  TORCH_CHECK(positions.numel() == T && slots.numel() == T);
  TORCH_CHECK(qkv.size(1) >= (H + G) * dk + G * dv, "qkv rows too short");
  TORCH_CHECK(act_kind(k_cache, "k_cache") == f && act_kind(v_cache, "v_cache") == f);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == dk && v_cache.size(1) == G && v_cache.size(3) == dv &&
              v_cache.size(0) == k_cache.size(0) && v_cache.size(2) == k_cache.size(2), "cache geometry");
  int rd = 0;
  const float* cs = nullptr;
  if (cos_sin.has_value()) {
    check_f32(*cos_sin, "cos_sin");
    TORCH_CHECK(cos_sin->dim() == 2);
    rd = (int)cos_sin->size(1);
    cs = cos_sin->data_ptr<float>();
  }
  check_rc(dgi_qk_prep(qkv.data_ptr(), f, T, (int)qkv.stride(0), positions.data_ptr<int>(), slots.data_ptr<int>(),
                       qw.data_ptr<float>(), kw.data_ptr<float>(), (float)eps, cs, rd, (int)H, (int)G, (int)dk, (int)dv,
                       k_cache.data_ptr(), v_cache.data_ptr(), (int)k_cache.size(2), full ? 1 : 0, half ? 1 : 0, cur_stream()),
           "qk_prep");
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(dgi, m) {
  m.def("dyt(Tensor(a!) y, Tensor x, Tensor alpha, Tensor w, Tensor b) -> ()");
  m.def("dyt_add(Tensor(a!) res, Tensor h, Tensor alpha1, Tensor w1, Tensor b1, Tensor ls, Tensor(b!)? y, "
        "Tensor? alpha2, Tensor? w2, Tensor? b2) -> ()");
  m.def("embed_dyt(Tensor(a!) res, Tensor ids, Tensor table, float scale, Tensor alpha, Tensor w, Tensor b) -> ()");
  m.def("qknorm_rope_cache(Tensor(a!) qkv, Tensor positions, Tensor slots, Tensor qw, Tensor kw, float eps, "
        "Tensor? cos_sin, int H, int G, int dk, int dv, Tensor(b!) k_cache, Tensor(c!) v_cache, float qt_coef=0.0, "
        "int qt_every=0) -> ()");
  m.def("linear_scan(Tensor(a!) y, int mode, Tensor q, Tensor k, Tensor v, Tensor aux1, Tensor? aux2, Tensor? par1, Tensor? par2, "
        "Tensor(b!) state, Tensor(c!)? norm, Tensor(d!)? mx, Tensor positions, Tensor seq_row0, Tensor seq_slots, int H, int G, "
        "int dk, int dv, float cap) -> ()");
  m.def("token_shift(Tensor(a!) out, Tensor h, Tensor mu, Tensor(b!) tail, Tensor positions, Tensor row_seq, Tensor seq_row0, "
        "Tensor seq_slots) -> ()");
  m.def("head_norm_gate(Tensor(a!) out, Tensor y, Tensor z, Tensor w, int heads, float eps, int sigmoid_gate) -> ()");
  m.def("rms_pair_mean(Tensor(a!) out, Tensor a, Tensor b, Tensor wa, Tensor wb, float eps) -> ()");
  m.def("qk_prep(Tensor(a!) qkv, Tensor positions, Tensor slots, Tensor qw, Tensor kw, float eps, Tensor? cos_sin, int H, int G, "
        "int dk, int dv, Tensor(b!) k_cache, Tensor(c!) v_cache, bool full, bool half) -> ()");
  m.def("masked_attn_rows(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_tables, "
        "Tensor? cu_seqlens, Tensor positions, int H, int G, float scale, int mask, Tensor? gate, "
        "Tensor? dist_bias=None, float softcap=0.0, Tensor? sinks=None) -> ()");
  m.def("paged_prefill_masked(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_tables, "
        "Tensor cu_seqlens_q, Tensor context_lens, Tensor tiles, int nh, int nkv, float scale, int mask, "
        "Tensor? gate, Tensor? dist_bias=None, float softcap=0.0, Tensor? sinks=None) -> ()");
  m.def("glu_clamped(Tensor(a!) out, Tensor gu, float limit, float alpha) -> ()");
  m.def("scale_softcap(Tensor(a!) out, Tensor x, float scale, float cap) -> ()");
  m.def("embed_streams(Tensor(a!) xs, Tensor ids, Tensor positions, Tensor row_seq, Tensor seq_row0, Tensor seq_slots, "
        "Tensor(b!) prev_tok, Tensor embed, Tensor? bigram, Tensor? pos_table, int buckets, int mul_prev, int mul_cur) -> ()");
  m.def("hc_mix_norm(Tensor(a!) xs, Tensor? y, Tensor? gate, Tensor? gate_b, Tensor? mix, Tensor? out, Tensor? in_next, "
        "Tensor? norm_w, float eps, Tensor(b!)? h32, Tensor(c!)? hd) -> ()");
  m.def("causal_conv(Tensor(a!) out, Tensor x, Tensor w, Tensor? bias, Tensor(b!)? tail, Tensor positions, Tensor row_seq, "
        "Tensor seq_row0, Tensor seq_slots, int act, bool residual) -> ()");
  m.def("ssm_scan(Tensor(a!) y, Tensor xbc, Tensor dt_raw, Tensor dt_bias, Tensor a_log, Tensor d_skip, Tensor(b!) state, "
        "Tensor positions, Tensor seq_row0, Tensor seq_slots, int heads, int dv, int N, int G, Tensor(c!)? ws=None, "
        "Tensor(d!)? wsd=None, int L=0, int nchunks=0) -> ()");
  m.def("gated_group_norm(Tensor(a!) out, Tensor y, Tensor z, Tensor w, int groups, float eps) -> ()");
  m.def("moe_route(Tensor(a!) idx, Tensor(b!) wts, Tensor logits, Tensor? correction, int sigmoid=0) -> ()");
  m.def("glu_rows(Tensor(a!) out, Tensor gu, int kind, float limit, float alpha, Tensor? row_scale) -> ()");
  m.def("stream_add_norm(Tensor(a!) x, Tensor? y, Tensor? post_w, Tensor? next_w, float eps, Tensor(b!)? out, "
        "Tensor? y2=None) -> ()");
  m.def("latent_prep(Tensor(a!) cq, Tensor proj, int q_rank, int kv_rank, int rot_dim, Tensor dq_w, Tensor? dkv_w, float eps, "
        "Tensor positions, Tensor slots, Tensor? cos_sin, bool interleaved, Tensor(b!)? cache) -> ()");
  m.def("latent_attn_rows(Tensor(a!) out, Tensor q, Tensor q_lat, Tensor cache, Tensor block_tables, Tensor? cu_seqlens, "
        "Tensor positions, int H, int dim, int rot_dim, int kv_rank, float scale, int window, Tensor? cos_sin, "
        "bool interleaved, int nsplit=1, Tensor(b!)? part_o=None, Tensor(c!)? part_ml=None, bool mfma=False) -> ()");
  m.def("rotate_heads(Tensor(a!) x, Tensor positions, Tensor cos_sin, bool interleaved, int H, int head_size, int offset) -> ()");
  m.def("gate_heads(Tensor(a!) out, Tensor ov, Tensor? gate, bool per_head) -> ()");
  m.def("gelu_tanh(Tensor(a!) out, Tensor x, Tensor? table, Tensor? ids, int col0) -> ()");
  m.def("glu_silu(Tensor(a!) out, Tensor gu) -> ()");
  m.def("moe_expert_gate_up(Tensor(a!) mid, Tensor h, Tensor idx, Tensor gate_up, Tensor? pair_scale=None, int act=0, "
        "float limit=0.0, float alpha=1.702) -> ()");
  m.def("moe_expert_down(Tensor(a!) ys, Tensor mid, Tensor idx, Tensor down) -> ()");
  m.def("moe_combine(Tensor(a!) out, Tensor ys, Tensor? where, Tensor h, Tensor idx, Tensor? wts, Tensor? shared, int E) -> ()");
}

TORCH_LIBRARY_IMPL(dgi, CUDA, m) {
  m.impl("dyt", &dyt);
  m.impl("dyt_add", &dyt_add);
  m.impl("embed_dyt", &embed_dyt);
  m.impl("qknorm_rope_cache", &qknorm_rope_cache);
  m.impl("linear_scan", &linear_scan);
  m.impl("token_shift", &token_shift);
  m.impl("head_norm_gate", &head_norm_gate);
  m.impl("rms_pair_mean", &rms_pair_mean);
  m.impl("qk_prep", &qk_prep);
  m.impl("masked_attn_rows", &masked_attn_rows);
  m.impl("paged_prefill_masked", &paged_prefill_masked);
  m.impl("glu_clamped", &glu_clamped);
  m.impl("scale_softcap", &scale_softcap);
  m.impl("embed_streams", &embed_streams);
  m.impl("hc_mix_norm", &hc_mix_norm);
  m.impl("causal_conv", &causal_conv);
  m.impl("ssm_scan", &ssm_scan);
  m.impl("gated_group_norm", &gated_group_norm);
  m.impl("moe_route", &moe_route);
  m.impl("glu_rows", &glu_rows);
  m.impl("stream_add_norm", &stream_add_norm);
  m.impl("latent_prep", &latent_prep);
  m.impl("latent_attn_rows", &latent_attn_rows);
  m.impl("rotate_heads", &rotate_heads);
  m.impl("gate_heads", &gate_heads);
  m.impl("gelu_tanh", &gelu_tanh);
  m.impl("glu_silu", &glu_silu);
  m.impl("moe_expert_gate_up", &moe_expert_gate_up);
  m.impl("moe_expert_down", &moe_expert_down);
  m.impl("moe_combine", &moe_combine);
}
