// attention_decode.hip's kernel for scores with a cap, a distance bias or a query temperature.
#include "attention_decode_kernel.h"

int launch_attention_decode_scores(const AttentionDecodeArgs& args, hipStream_t stream) {
  switch (args.m.base.hd) {
#define TS_CASE(HD) case HD: return launch_decode<HD, true>(args, stream);
    TS_CASE(16) TS_CASE(32) TS_CASE(48) TS_CASE(64) TS_CASE(80) TS_CASE(96) TS_CASE(112)
    TS_CASE(128) TS_CASE(144) TS_CASE(160) TS_CASE(176) TS_CASE(192) TS_CASE(208) TS_CASE(224)
    TS_CASE(240) TS_CASE(256)
#undef TS_CASE
    default: TS_FAIL("attention_decode: head_dim=%d not built", args.m.base.hd);
  }
}
