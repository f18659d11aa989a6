// dgi/csrc/mix/masked_prefill.hip — the MFMA varlen flash-attention kernel of
// prefill_attention.hip instantiated with a block mask and a sigmoid output gate
// and optionally a learned distance bias (prefill_attention_kernel.h, MASKED = true, BIAS): prompt portions of mixers whose bf16 key and
// value heads share one size of 64 or 128.  Other geometries and fp32 run masked_attention.hip.
//
// grid = (query tiles of 128 rows, heads); K/V tiles of 64 keys staged through two LDS stages;
// a workgroup starts at the tile that holds the first block of its first row, so the work per
// query row is bounded by the block size, not by the context.
#include "../prefill_attention_kernel.h"

using namespace dgi;
using namespace dgi::prefill;

// tiles: int32 [n_tiles, 2] = (sequence index, first query row of the 128-row tile);
// mask: block size in positions (0 = plain causal, < 0: a sliding window of -mask positions); gate: [rows, >= nh * hd] or nullptr;
// softcap > 0: scores capped at softcap * tanh(s / softcap); sinks: [nh] fp32 logits that join the denominator, or nullptr
extern "C" int dgi_paged_prefill_masked(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                        const int* block_tables, int bt_stride, const int* cu_seqlens_q,
                                        const int* context_lens, const int* tiles, int n_tiles, void* out,
                                        int out_stride, int nh, int nkv, int hd, int block_size, float scale,
                                        int mask, const void* gate, int gate_stride, const float* dist_bias,
                                        int n_dist, float softcap, const float* sinks, hipStream_t s) {
  if (n_tiles == 0) return 0;
  if (hd != 128 && hd != 64) return -5;
  if (nkv <= 0 || nh % nkv) return -2;
  if (dist_bias && (n_dist < 1 || scale == 0.f)) return -6;
  int bs_log2 = 0;
  while ((1 << bs_log2) < block_size) ++bs_log2;
  if ((1 << bs_log2) != block_size) return -4;
  const float scale_log2 = scale * 1.4426950408889634f;
#define DGI_PREFILL_MASKED(HDV, BIASV)                                                                   \
  prefill_attn_kernel<HDV, 4, 1, true, BIASV><<<dim3(n_tiles, nh), 256, 0, s>>>(                          \
      (const uint16_t*)q, q_stride, (const uint16_t*)k_cache, (const uint16_t*)v_cache, block_tables,     \
      bt_stride, cu_seqlens_q, context_lens, tiles, (uint16_t*)out, out_stride, nh, nkv, bs_log2,         \
      scale_log2, nullptr, 0, mask, (const uint16_t*)gate, gate_stride, dist_bias, n_dist, 1.f / scale,         \
      softcap, sinks)
  if (dist_bias) {
    if (hd == 128) DGI_PREFILL_MASKED(128, true);
    else DGI_PREFILL_MASKED(64, true);
  } else {
    if (hd == 128) DGI_PREFILL_MASKED(128, false);
    else DGI_PREFILL_MASKED(64, false);
  }
#undef DGI_PREFILL_MASKED
  DGI_CHECK_LAUNCH();
  return 0;
}
