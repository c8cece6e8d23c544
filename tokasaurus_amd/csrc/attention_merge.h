// Merging the partial results that the attention kernel leaves when the keys of a tile are cut
// into splits, done by the workgroup that needs the merged rows as the operand of the output
// product: every thread of the workgroup takes (token, 4 columns) items, asks for all the
// splits' values at once, adds them in split order, and writes bfloat16 into LDS in the order in
// which the matrix core's lanes read their operand: the 8 values of (step of 32 columns,
// lane = quarter * 16 + token) lie together.  One token a request, each a tile of its own
// (decode): the partial results of request t, kv head h, split s start at item
// (t * nkv + h) * max_splits + s, 16 rows of D (and of 2: maximum in units of log 2, sum) each.
#pragma once

#include "common.h"

struct MergeArgs {
  const float* part_o;   // [tokens][nkv][max_splits][16][D]
  const float* part_ml;  // [tokens][nkv][max_splits][16][2]
  const int* kv_len;     // [tokens] keys of each request
  int M, nq, nkv, D;
  int split, max_splits, window;
};

#define TK_MERGE_UNROLL 16  // splits whose values are in flight together

__device__ __forceinline__ uint16_t merge_bf16_bits(float v) {
  union { bf16_t h; uint16_t u; } x;
  x.h = __float2bfloat16(v);
  return x.u;
}

// stage: LDS of ((nq * D + 31) / 32) * 64 * 8 bfloat16.  Rows of tokens past M are left as they
// are (they reach no output that is kept); the columns past nq * D of the last step are zeroed
// (their weights are zero, and 0 * garbage may be NaN).  The caller synchronises the workgroup.
__device__ __forceinline__ void merge_attention_to_lds(const MergeArgs& m, bf16_t* stage, int n_threads) {
  const int D = m.D, group = m.nq / m.nkv, K = m.nq * D;
  const int K32 = (K + 31) >> 5;
  for (int it = threadIdx.x; it < 16 * (K32 * 32 - K) / 4; it += n_threads) {
    const int token = it & 15, k = K + (it >> 4) * 4;
    *(uint64_t*)(stage + ((size_t)((k >> 5) * 64 + ((k & 31) >> 3) * 16 + token) * 8 + (k & 7))) = 0;
  }
  const int chunks = K / 4;  // K is a multiple of 8
  for (int it = threadIdx.x; it < m.M * chunks; it += n_threads) {
    const int token = it / chunks, k = (it - token * chunks) * 4;
    const int head = k / D, c0 = k - head * D;
    const int kvh = head / group, row = head - kvh * group;
    const int kvl = m.kv_len[token];
    const int lo = m.window > 0 ? max(0, kvl - m.window) : 0;
    const int s_first = lo / m.split, nsp = (kvl - 1) / m.split - s_first + 1;
    const size_t item0 = ((size_t)token * m.nkv + kvh) * m.max_splits;
    const float* ml = m.part_ml + (item0 * 16 + row) * 2;
    const float* po = m.part_o + (item0 * 16 + row) * D + c0;
    float mx = -INFINITY, l = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
    // blocks of TK_MERGE_UNROLL splits (one block with the splits the engine plans): within a
    // block everything is asked for at once; from block to block the running maximum is carried
    // and what was summed is rescaled, always in split order
    for (int base = 0; base < nsp; base += TK_MERGE_UNROLL) {
      union { uint64_t u; float f[2]; } mlv[TK_MERGE_UNROLL], pa[TK_MERGE_UNROLL], pb[TK_MERGE_UNROLL];
#pragma unroll
      for (int j = 0; j < TK_MERGE_UNROLL; ++j) {
        if (base + j < nsp) {
          mlv[j].u = *(const uint64_t*)(ml + (size_t)(base + j) * 32);
          pa[j].u = *(const uint64_t*)(po + (size_t)(base + j) * 16 * D);
          pb[j].u = *(const uint64_t*)(po + (size_t)(base + j) * 16 * D + 2);
        }
      }
      float m_new = mx;
#pragma unroll
      for (int j = 0; j < TK_MERGE_UNROLL; ++j)
        if (base + j < nsp) m_new = fmaxf(m_new, mlv[j].f[0]);
      const float keep = mx == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mx - m_new);
      l *= keep;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] *= keep;
      mx = m_new;
#pragma unroll
      for (int j = 0; j < TK_MERGE_UNROLL; ++j) {
        if (base + j < nsp) {
          const float w = mlv[j].f[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mlv[j].f[0] - mx);
          l += w * mlv[j].f[1];
          o[0] += w * pa[j].f[0];
          o[1] += w * pa[j].f[1];
          o[2] += w * pb[j].f[0];
          o[3] += w * pb[j].f[1];
        }
      }
    }
    const float inv = 1.0f / l;
    union { uint64_t u; uint16_t h[4]; } pk;
#pragma unroll
    for (int j = 0; j < 4; ++j) pk.h[j] = merge_bf16_bits(o[j] * inv);
    const int step = k >> 5, qq = (k & 31) >> 3;
    *(uint64_t*)(stage + ((size_t)(step * 64 + qq * 16 + token) * 8 + (k & 7))) = pk.u;
  }
}
