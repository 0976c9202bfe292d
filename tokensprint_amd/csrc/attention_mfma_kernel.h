// The kernel of attention_mfma.hip as a template, so that its forms with and without
// score extras compile in translation units of their own, side by side.
#pragma once
#include "attention_core.h"

int launch_attention_merge(const AttentionMfmaArgs& args, hipStream_t stream);

// COOP = false: a wavefront per item walks its keys alone.
// COOP = true: a workgroup per item; its four waves take every fourth 32-key block and
// merge in LDS (few tiles: decode), so a short context costs one round of loads.
// EXTRA: scores with a cap, a distance bias or a query temperature (attention.h).
template <int HD, bool COOP, bool PAGE16, bool EXTRA>
__global__ __launch_bounds__(256, HD <= 128 ? 2 : 1) void attention_mfma_kernel(AttentionMfmaArgs args) {
  constexpr int DB = HD / 16;
  const AttentionArgs& a = args.base;
  const int wave = uniform(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  const int items = args.num_tiles * a.nkv * args.head_blocks;
  const int item = COOP ? blockIdx.x : blockIdx.x * 4 + wave;
  if (item >= items) return;
  const int tile = item / (a.nkv * args.head_blocks);
  const int kvh = (item / args.head_blocks) % a.nkv;
  const int hb = item % args.head_blocks;
  const int split = blockIdx.y;
  // without a tile list every entry brings one token (a decode step): tile = entry = token
  const int entry = args.tiles ? uniform(args.tiles[tile * 3]) : tile,
            tok0 = args.tiles ? uniform(args.tiles[tile * 3 + 1]) : tile,
            ntok = args.tiles ? uniform(args.tiles[tile * 3 + 2]) : 1;
  const int* table = a.table + (int64_t)entry * a.table_width;

  // my query row: column r of S^T
  const int ti = r / args.rows_per_token;
  const int hh = hb * 16 + r % args.rows_per_token;          // head inside the group
  const bool row_ok = ti < ntok && hh < group;
  const int token = tok0 + min(ti, ntok - 1);
  const int head = kvh * group + min(hh, group - 1);

  // key range of the tile and my share of its chunks
  const int pos_first = uniform(a.positions[tok0]);           // positions are consecutive
  const int pos_last = pos_first + ntok - 1;
  const int lo_tile = first_visible(a, pos_first);
  const int c_first = lo_tile / kChunk, c_last = pos_last / kChunk;
  const int per = (c_last - c_first + args.num_splits) / args.num_splits;   // ceil(n / splits)
  const int c0 = c_first + split * per, c1 = min(c0 + per, c_last + 1);
  if (c0 > c_last) {   // more splits than chunks: a neutral partial, no data touched
    if (g == 0 && (!COOP || wave == 0)) {
      const int64_t slot = ((int64_t)item * args.num_splits + split) * 16 + r;
      args.partial_ml[slot * 2] = -INFINITY;
      args.partial_ml[slot * 2 + 1] = 0.f;
    }
    return;
  }

  TileState<HD> t;
  t.pos = row_ok ? pos_first + ti : -1;
  t.lo = first_visible(a, t.pos);
  load_query<HD>(t, (const bf16_t*)a.q + ((int64_t)token * a.nq + head) * HD, row_ok, g);
  const float scale_log2 = a.scale * 1.44269504088896341f;
  ScoreExtra x;
  if (EXTRA) x = score_extra(a, head, t.pos);
  const int lo_last = first_visible(a, pos_last);

  constexpr int kStride = COOP ? 128 : 32;
  const int key_begin = max(c0 * kChunk, lo_tile & ~31) + (COOP ? wave * 32 : 0);
  const int key_end = min(c1 * kChunk, pos_last + 1);
  PageCursor cur{(ConstTable)table, a.page_size, pos_last, -1, -1};
  if (PAGE16) cur.start(key_begin);

  KvBlock<HD> A, B;
  // head sizes in whole 32-element slices on power-of-two pages take the blocks with
  // 16-byte value loads (the keys of a block permuted over the score products' rows)
  constexpr bool kWide = PAGE16 && HD % 32 == 0;
  auto load_block = [&](KvBlock<HD>& b, int kb) {
    if constexpr (kWide) load_kv_block_wide<HD>(b, a, cur, kvh, kb, kStride, r, g);
    else load_kv_block<HD, PAGE16>(b, a, table, cur, kvh, kb, kStride, r, g);
  };
  if (key_begin < key_end) load_block(A, key_begin);
  for (int kb = key_begin; kb < key_end; kb += 2 * kStride) {
    if (kb + kStride < key_end) load_block(B, kb + kStride);
    tile_update<HD, false, kWide, EXTRA>(t, A, kb, scale_log2, kb + 31 <= pos_first && kb >= lo_last, g, &x);
    if (kb + kStride >= key_end) break;
    if (kb + 2 * kStride < key_end) load_block(A, kb + 2 * kStride);
    tile_update<HD, false, kWide, EXTRA>(t, B, kb + kStride, scale_log2,
                                         kb + kStride + 31 <= pos_first && kb + kStride >= lo_last, g, &x);
  }
  f32x4 (&o)[DB] = t.o;
  float m = t.m, l = row_sum<HD>(t);

  if (COOP) {   // the four waves' partial results, merged by wave 0 in wave order
    __shared__ float s_ml[3][kWave][2];
    __shared__ f32x4 s_o[3][DB][kWave];
    if (wave > 0) {
      s_ml[wave - 1][lane][0] = m;
      s_ml[wave - 1][lane][1] = l;
#pragma unroll
      for (int db = 0; db < DB; ++db) s_o[wave - 1][db][lane] = o[db];
    }
    __syncthreads();
    if (wave > 0) return;
    float M = m;
#pragma unroll
    for (int w = 0; w < 3; ++w) M = fmaxf(M, s_ml[w][lane][0]);
    if (M != -INFINITY) {
      const float w0 = __builtin_amdgcn_exp2f(m - M);
      l *= w0;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[db][i] *= w0;
#pragma unroll
      for (int w = 0; w < 3; ++w) {
        const float mw = s_ml[w][lane][0];
        if (mw == -INFINITY) continue;
        const float ww = __builtin_amdgcn_exp2f(mw - M);
        l += s_ml[w][lane][1] * ww;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const f32x4 ow = s_o[w][db][lane];
#pragma unroll
          for (int i = 0; i < 4; ++i) o[db][i] += ow[i] * ww;
        }
      }
      m = M;
    }
  }

  // lane (r, g) holds O^T[d = db*16 + g*4 + i][row r]
  if (args.num_splits == 1) {
    if (!row_ok) return;
    store_tile<HD>(t, sum_with_sink(l, m, a.sink, head), (bf16_t*)a.out + ((int64_t)token * a.nq + head) * HD, g);
  } else {
    const int64_t slot = ((int64_t)item * args.num_splits + split) * 16 + r;
    if (row_ok) {
      float* po = args.partial_o + slot * HD;
#pragma unroll
      for (int db = 0; db < DB; ++db) *(f32x4*)(po + db * 16 + g * 4) = o[db];
    }
    if (g == 0) {
      args.partial_ml[slot * 2] = m;      // in units of log2: scores were scaled by log2(e)
      args.partial_ml[slot * 2 + 1] = l;
    }
  }
}

template <int HD, bool EXTRA>
static int launch_mfma(const AttentionMfmaArgs& args, hipStream_t stream) {
  const int items = args.num_tiles * args.base.nkv * args.head_blocks;
  const int P = args.base.page_size;
  const bool page16 = P >= 16 && (P & (P - 1)) == 0;
  const dim3 coop_grid(items, args.num_splits), walk_grid((items + 3) / 4, args.num_splits);
  if (args.cooperative && page16)
    hipLaunchKernelGGL((attention_mfma_kernel<HD, true, true, EXTRA>), coop_grid, dim3(256), 0, stream, args);
  else if (args.cooperative)
    hipLaunchKernelGGL((attention_mfma_kernel<HD, true, false, EXTRA>), coop_grid, dim3(256), 0, stream, args);
  else if (page16)
    hipLaunchKernelGGL((attention_mfma_kernel<HD, false, true, EXTRA>), walk_grid, dim3(256), 0, stream, args);
  else
    hipLaunchKernelGGL((attention_mfma_kernel<HD, false, false, EXTRA>), walk_grid, dim3(256), 0, stream, args);
  if (args.num_splits > 1) return launch_attention_merge(args, stream);
  return 0;
}

