// The LDS-sharing kernel for long portions with scores that have a cap, a distance bias or a
// query temperature: every head size, items of four tiles.
#include "attention_prefill_lds_kernel.h"

int launch_attention_prefill_scores(const AttentionMfmaArgs& args, hipStream_t stream) {
  const int items = args.num_tiles * args.base.nkv * args.head_blocks;
  switch (args.base.hd) {
#define TS_CASE(HD) case HD: hipLaunchKernelGGL((attention_prefill_lds_kernel<HD, true>), dim3(items), dim3(256), 0, stream, args); return 0;
    TS_CASE(16) TS_CASE(32) TS_CASE(48) TS_CASE(64) TS_CASE(80) TS_CASE(96) TS_CASE(112)
    TS_CASE(128) TS_CASE(144) TS_CASE(160) TS_CASE(176) TS_CASE(192) TS_CASE(208) TS_CASE(224)
    TS_CASE(240) TS_CASE(256)
#undef TS_CASE
    default: TS_FAIL("attention_prefill: head_dim=%d not built", args.base.hd);
  }
}
