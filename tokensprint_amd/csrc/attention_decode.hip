// Paged attention for a decode step (one new token per batch entry) on the matrix cores,
// bfloat16, page sizes that are powers of two from 16 up.
//
// One workgroup owns a tile: the query heads of one key/value head of one entry (up to
// 16 rows) and, with `num_splits` > 1, one share of the entry's 128-key chunks.  Its NW
// waves take every NW-th block of 32 keys with the loads and arithmetic of
// attention_core.h and merge in LDS, so up to a few thousand keys cost one launch and no
// partial results in memory; longer contexts are split over workgroups and merged by
// attention_merge, or by the workgroup of the item that finishes last (below).
//
// Fused form (FUSED): what lies between the q/k/v projection and attention happens here
// as well, so a decode layer needs no kernel for it.  Every wave reads its query rows
// from the projection's output, applies the per-head RMSNorm and the rotation in float32
// in the registers of the operand layout (a head's four lanes hold a quarter of it each;
// the rotation's partner of element d, d +- hd/2, is in the lane 32 further), and rounds
// to bfloat16 as the unfused kernel stores it.  The last wave of a workgroup does this
// for the others instead of walking (they have their first key block in flight and no
// registers to spare) and hands the rows over in LDS.  In the first split's workgroup it
// also prepares the new key, writes key and value to their cache slot and gives them to
// the merge as one more partial sum (score q.k, weight 1, value v) instead of anyone
// reading them back; the keys walked from the cache end one before the new position.
// (A wave of its own also because a store in flight makes every later wait for a load a
// wait for all of them: loads and stores share one counter.)
#include "attention_decode_kernel.h"

int ts_check_attention_mfma_args(const AttentionMfmaArgs& args, const char* who);
int launch_attention_decode_scores(const AttentionDecodeArgs& args, hipStream_t stream);

// 1 if ts_attention_decode takes this head size and page size (fused: its fused form).
extern "C" int ts_attention_decode_fits(int hd, int page_size, int fused) {
  if (hd < 16 || hd > 256 || hd % 16 || (fused && hd % 32)) return 0;
  return page_size >= 16 && (page_size & (page_size - 1)) == 0;
}

extern "C" int ts_attention_decode(const AttentionDecodeArgs* p, hipStream_t stream) {
  AttentionDecodeArgs args = *p;
  const AttentionMfmaArgs& m = args.m;
  const AttentionArgs& a = m.base;
  if (a.num_tokens <= 0) return 0;
  if (ts_check_attention_mfma_args(m, "attention_decode")) return -1;
  if (m.tiles || m.num_tiles != a.num_tokens || a.num_tokens != a.num_entries)
    TS_FAIL("attention_decode: one token per entry and no tile list (tokens %d, entries %d)",
            a.num_tokens, a.num_entries);
  if (!ts_attention_decode_fits(a.hd, a.page_size, args.qkv != nullptr))
    TS_FAIL("attention_decode: head_dim=%d, page_size=%d not served", a.hd, a.page_size);
  if (m.num_splits < 1 || m.num_splits > 65535) TS_FAIL("attention_decode: num_splits=%d", m.num_splits);
  if (m.num_splits > 1 && (!m.partial_o || !m.partial_ml))
    TS_FAIL("attention_decode: splits need partial buffers");
  if (args.qkv) {
    if ((uintptr_t)args.qkv & 15) TS_FAIL("attention_decode: qkv must be 16-byte aligned");
    if (args.row_extra < 0 || args.row_extra % 8) TS_FAIL("attention_decode: row_extra=%d must be a multiple of 8", args.row_extra);
    if ((args.cos == nullptr) != (args.sin == nullptr)) TS_FAIL("attention_decode: cos and sin go together");
    if (args.kv_in_row != 0 && args.kv_in_row != a.nkv)
      TS_FAIL("attention_decode: the row brings %d key heads, the cache has %d", args.kv_in_row, a.nkv);
  } else if (!a.q) {
    TS_FAIL("attention_decode: neither q nor qkv");
  }
  int rc = 0;
  if (has_score_extras(a)) {
    if (launch_attention_decode_scores(args, stream)) return -1;
    TS_CHECK_LAUNCH("attention_decode");
    return 0;
  }
  switch (a.hd) {
#define TS_CASE(HD) case HD: rc = launch_decode<HD, false>(args, stream); break;
    TS_CASE(16) TS_CASE(32) TS_CASE(48) TS_CASE(64) TS_CASE(80) TS_CASE(96) TS_CASE(112)
    TS_CASE(128) TS_CASE(144) TS_CASE(160) TS_CASE(176) TS_CASE(192) TS_CASE(208) TS_CASE(224)
    TS_CASE(240) TS_CASE(256)
#undef TS_CASE
    default: TS_FAIL("attention_decode: head_dim=%d not built", a.hd);
  }
  if (rc) return rc;
  TS_CHECK_LAUNCH("attention_decode");
  return 0;
}
