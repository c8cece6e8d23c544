// Paged attention on the gfx950 matrix cores, bfloat16 storage, 32-bit softmax.
// One kernel serves prompt portions and single decoded tokens.
//
// Rows.  For a request and a kv head, the rows are the pairs (token of this step,
// query head of the kv head's group), numbered token * group + head, and cut into
// row tiles of 16.  A wavefront owns RT row tiles of one request and walks the keys
// they may see in steps of 32.  With the keys as the first operand of
// v_mfma_f32_16x16x32_bf16 and the queries as the second,
//     S^T[key 4q+j][row r]  is element j of lane (r = lane % 16, q = lane / 16),
// so a lane holds, for ONE row, 4 keys of each 16-key block.  These 8 numbers
// are exactly what the lane must provide as the second operand of the product
// O^T = V^T P^T, if slot 8q+j of that product's inner index stands for key 4q+j
// of the first block and slot 8q+4+j for key 4q+j of the second.  A page keeps
// its values in groups of 4 tokens ([P / 4][d][4]), so the matching first operand
// is read with two 8-byte loads per lane, and its keys in pieces of 8 elements
// ([d / 8][P][8]), so that in both kinds of load 16 neighbouring lanes read
// consecutive memory: the vector cache handles a load at the rate of the cache
// lines it touches, not of its bytes.  Nothing passes through LDS.
// P is a power of two, at least 4.
//
// Two row tiles of a wavefront need not be neighbours: under a causal mask the host
// pairs an early tile of a prompt with a late one, so that every wavefront has the
// same number of (row tile, key step) products.  A row tile is skipped in the steps
// that none of its rows sees; steps that all of its rows see whole are not masked.
//
// Splits.  The keys of a wavefront's tiles are cut at absolute multiples of `split`;
// each (tile, kv head, split) is one workgroup of NW wavefronts, which cut the split's
// keys into NW consecutive parts (multiples of 32) and add their results through
// LDS in wavefront order.  A tile with one split writes the output; otherwise
// partial (max, sum, weighted values) go to scratch and a second kernel adds them
// in split order.  With few tiles (decode) many wavefronts with two or three steps
// each keep enough loads in flight; with many tiles (prompts) NW is 1.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

struct AttnArgs {
  const bf16_t* q;
  int q_stride;
  bf16_t* out;
  int out_stride;
  const bf16_t* kcache;
  const bf16_t* vcache;
  const int* block_table;
  int table_stride;
  const int* q_start;   // [requests + 1]
  const int* kv_len;    // [requests]
  const int* tile_req;  // [tiles]
  const int* tile_row0; // [tiles] first row of the wavefront's first row tile
  const int* tile_row1; // [tiles] first row of its second row tile, -1 for none; null: the 16 rows after the first
  int n_tiles;
  int nq, nkv, group, P, p_shift, window;
  float scale_log2;  // scale * log2(e) > 0
  int split;         // keys per split, a multiple of 32
  int max_splits;    // splits a tile may have (size of the scratch)
  float* part_o;     // [tiles][nkv][max_splits][16 * RT][D]
  float* part_ml;    // [tiles][nkv][max_splits][16 * RT][2]
};

// What a (wavefront's) tile covers.  Per row tile: rows row0 .. row0 + 15 (row0 < 0: none),
// keys [lo, hi] that some row sees and [full_lo, full_hi] that every row sees.
struct TileRange {
  int req, qs, qlen, kvl, n_rows, lo, hi, s_first, s_last;
  int row0[2], rt_lo[2], rt_hi[2], full_lo[2], full_hi[2];
};

__device__ __forceinline__ TileRange tile_range(const AttnArgs& a, int tile, int row_tiles) {
  TileRange t;
  t.req = a.tile_req[tile];
  t.qs = a.q_start[t.req];
  t.qlen = a.q_start[t.req + 1] - t.qs;
  t.kvl = a.kv_len[t.req];
  t.n_rows = t.qlen * a.group;
  t.row0[0] = a.tile_row0[tile];
  t.row0[1] = -1;
  if (row_tiles == 2) {
    t.row0[1] = a.tile_row1 ? a.tile_row1[tile] : t.row0[0] + 16;
    if (t.row0[1] >= t.n_rows) t.row0[1] = -1;
  }
  t.lo = 0x7fffffff;
  t.hi = -1;
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    t.rt_lo[rt] = t.full_lo[rt] = 0x7fffffff;
    t.rt_hi[rt] = t.full_hi[rt] = -1;
    if (t.row0[rt] < 0) continue;
    const int first_tok = t.row0[rt] / a.group;
    const int last_tok = min(t.row0[rt] + 15, t.n_rows - 1) / a.group;
    const int pos_first = t.kvl - t.qlen + first_tok, pos_last = t.kvl - t.qlen + last_tok;
    t.rt_hi[rt] = pos_last;
    t.rt_lo[rt] = a.window > 0 ? max(0, pos_first - a.window + 1) : 0;
    t.full_hi[rt] = pos_first;
    t.full_lo[rt] = a.window > 0 ? max(0, pos_last - a.window + 1) : 0;
    t.lo = min(t.lo, t.rt_lo[rt]);
    t.hi = max(t.hi, t.rt_hi[rt]);
  }
  t.s_first = t.lo / a.split;
  t.s_last = t.hi / a.split;
  return t;
}

// first <= x <= last as one unsigned comparison (an empty range, last < first, holds nothing)
struct Range {
  int first;
  unsigned span;
  __device__ __forceinline__ bool holds(int x) const { return (unsigned)(x - first) <= span; }
};
__device__ __forceinline__ Range range_of(int first, int last) {
  return last >= first ? Range{first, (unsigned)(last - first)} : Range{0x7fffffff, 0u};
}

// The maximum over the four lanes (r, 0..3) that share a row: lanes 16 and 32 apart,
// with the gfx950 swaps of 16-lane rows and of wavefront halves.
__device__ __forceinline__ float max_over_quarters(float x) {
  const unsigned u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float y = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const unsigned v = __float_as_uint(y);
  const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// The loads of one step of 32 keys.  Keys: lane (r, q) reads 8 values of key
// kb + 16 blk + r for every 32-wide step over the head size.  Values: lane (r, q)
// reads, for d = 16 dt + r, the 4 keys kb + 16 blk + 4q .. + 3.  Every address lies
// in a page of the tile's key range [lo, hi], so a load past the end reads valid
// memory (whose contents the masks keep out of the result).
template <int DT>
struct StepRegs {
  bf16x8_t kv[2][(DT + 1) / 2];
  union { bf16x4_t half[2]; uint32_t u[4]; bf16x8_t whole; } vv[DT];  // the two 16-key blocks side by side
};

// BIG: pages of 16 keys or more, so the 16 keys of a block lie in one page, which a
// scalar load looks up; the lane's part of the address is the same in every step.
// The pages of the two 16-key blocks of the step at `kb` (BIG only): looked up a step before
// the loads that need them are issued, so that no load waits for a table entry.
struct StepPages {
  int page[2];
};

__device__ __forceinline__ StepPages step_pages(const AttnArgs& a, const int* table, int kb, int lo, int hi) {
  const int sh = a.p_shift;
  StepPages p;
  p.page[0] = table[min(max(kb >> sh, lo >> sh), hi >> sh)];
  p.page[1] = table[min(max((kb + 16) >> sh, lo >> sh), hi >> sh)];
  return p;
}

template <int DT, bool BIG>
__device__ __forceinline__ void load_step(StepRegs<DT>& s, const AttnArgs& a, const int* table, const StepPages& pages,
                                          int kvh, int kb, int lo, int hi, int r, int q) {
  constexpr int D = DT * 16;
  constexpr int KS = (DT + 1) / 2;
  const int P = a.P, sh = a.p_shift;
  // the lane's own part of a key and of a value address inside any page of this kv head
  const unsigned lane_k = (unsigned)(kvh * P * D + r * 8);
  const unsigned lane_v = (unsigned)(kvh * P * D + (q * D + r) * 4);
#pragma unroll
  for (int blk = 0; blk < 2; ++blk) {
    const bf16_t* kp;
    const bf16_t* vp;
    if constexpr (BIG) {
      const int key0 = kb + blk * 16;
      // one 32 x 32 -> 64-bit product a page: the kv head's offset is in the lane's part already
      const size_t base = (size_t)(unsigned)pages.page[blk] * (unsigned)(a.nkv * P * D);
      const int in_page = key0 & (P - 1);
      kp = a.kcache + base + (unsigned)(in_page * 8) + lane_k;
      vp = a.vcache + base + (unsigned)((in_page >> 2) * (D * 4)) + lane_v;
    } else {
      const int kk = min(max(kb + blk * 16 + r, lo), hi);
      const int page = table[kk >> sh];
      kp = a.kcache + ((size_t)page * a.nkv + kvh) * ((size_t)P * D) + (size_t)(kk & (P - 1)) * 8;
      int kc = kb + blk * 16 + q * 4;
      if (kc > hi) kc = hi & ~3;
      if (kc + 3 < lo) kc = lo & ~3;
      const int vpage = table[kc >> sh];
      vp = a.vcache + ((size_t)vpage * a.nkv + kvh) * ((size_t)P * D) + (size_t)((kc & (P - 1)) >> 2) * (D * 4) + r * 4;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 32 + q * 8;  // piece d0 / 8 of the key
      if (d0 < D) {
        s.kv[blk][ks] = *(const bf16x8_t*)(kp + (size_t)(d0 >> 3) * P * 8);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) s.kv[blk][ks][e] = (__bf16)0.f;
      }
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) s.vv[dt].half[blk] = *(const bf16x4_t*)(vp + dt * 64);
  }
}

// Wavefronts a workgroup may have: the fewer, the more registers each has for loads in flight.
__host__ __device__ constexpr int max_waves(int dt, int rt) { return rt == 2 ? 4 : (dt <= 4 ? 16 : 8); }

// PF steps of loads are in flight: a lone wavefront on a long tile waits on memory otherwise.
template <int DT, int RT, bool BIG>
__global__ __launch_bounds__(64 * max_waves(DT, RT)) void paged_attention_mfma_kernel(AttnArgs a) {
  extern __shared__ __align__(16) float wg_part[];  // [wavefront][16 * RT rows][D + 4], when NW > 1
  constexpr int D = DT * 16;
  constexpr int KS = (DT + 1) / 2;  // 32-wide steps over the head size
  constexpr int PF = RT == 1 ? 2 : 3;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int NW = blockDim.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  // Workgroups go to the chip's eight dies in turn, each with a cache of its own.  Prompts
  // (two row tiles): kv head fastest, so a die serves few kv heads and keeps their keys and
  // values, which every tile of the request reads again, to itself.  Decoded tokens read
  // their keys once: tile fastest, as measured.
  const int kvh = RT == 2 ? blockIdx.x % a.nkv : blockIdx.x / a.n_tiles;
  const int tile = RT == 2 ? blockIdx.x / a.nkv : blockIdx.x % a.n_tiles;
  const TileRange t = tile_range(a, tile, RT);
  const int s = t.s_first + blockIdx.z;
  if (s > t.s_last) return;
  const int nsp = t.s_last - t.s_first + 1;
  // this wavefront's part of the split: `sub` keys, a multiple of 32
  const int sub = a.split / NW;
  const int k_begin = max((t.lo >> 5) << 5, s * a.split + wave * sub);
  const int k_end = min(t.hi + 1, s * a.split + (wave + 1) * sub);
  const int* table = a.block_table + (size_t)t.req * a.table_stride;

  // the steps (by their first key) in which a row tile has a row that sees a key, in which all
  // of its rows see all 32 keys, and in which all 32 keys lie in the tile's range
  Range active[RT], unmasked[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    active[rt] = range_of(t.rt_lo[rt] - 31, t.rt_hi[rt]);
    unmasked[rt] = range_of(t.full_lo[rt], t.full_hi[rt] - 31);
  }
  const Range inside = range_of(t.lo, t.hi - 31);

  // this lane's row in each of the RT tiles
  int pos_r[RT], lo_r[RT], flat_r[RT];
  bf16x8_t qv[RT][KS];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int flat = t.row0[rt] >= 0 ? t.row0[rt] + r : t.n_rows;
    const bool valid = flat < t.n_rows;
    flat_r[rt] = valid ? flat : -1;
    const int fl = valid ? flat : t.n_rows - 1;
    const int tok = fl / a.group, g = fl - tok * a.group;
    const int pos = t.kvl - t.qlen + tok;
    pos_r[rt] = valid ? pos : -1;
    lo_r[rt] = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    const bf16_t* qp = a.q + (size_t)(t.qs + tok) * a.q_stride + (size_t)(kvh * a.group + g) * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 32 + q * 8;
      if (d0 < D) {
        qv[rt][ks] = *(const bf16x8_t*)(qp + d0);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) qv[rt][ks][e] = (__bf16)0.f;
      }
    }
  }

  float m_run[RT], l_run[RT];  // running maximum of the row's products and sum of this lane's keys
  f32x4_t acc[RT][DT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    m_run[rt] = -INFINITY;
    l_run[rt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[rt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  auto compute_step = [&](StepRegs<DT>& cur, const int kb) {
    if (!inside.holds(kb)) {
      // values of keys outside the tile's range may be anything (a freed page): make them
      // zero by masking their 16 bits
      uint32_t keep[4];
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int key = kb + blk * 16 + q * 4 + 2 * h;
          const uint32_t lo16 = (key >= t.lo && key <= t.hi) ? 0x0000ffffu : 0u;
          const uint32_t hi16 = (key + 1 >= t.lo && key + 1 <= t.hi) ? 0xffff0000u : 0u;
          keep[blk * 2 + h] = lo16 | hi16;
        }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) cur.vv[dt].u[i] &= keep[i];
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if (!active[rt].holds(kb)) continue;  // none of the tile's rows sees these keys
      f32x4_t st[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        st[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.kv[0][ks], qv[rt][ks], st[0], 0, 0, 0);
        st[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.kv[1][ks], qv[rt][ks], st[1], 0, 0, 0);
      }
      // scores stay as the products are (scale_log2 > 0 keeps their order); the scale goes
      // into the exponent's multiply-add
      float sc[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) sc[e] = st[e >> 2][e & 3];
      if (!unmasked[rt].holds(kb)) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int key = kb + (e >> 2) * 16 + q * 4 + (e & 3);
          if (!(key >= lo_r[rt] && key <= pos_r[rt])) sc[e] = -INFINITY;
        }
      }
      float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
      mx = max_over_quarters(mx);
      const float m_new = fmaxf(m_run[rt], mx);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float mc = m_use * a.scale_log2;
      if (__any(m_new > m_run[rt])) {
        // some row's maximum moved: weigh what was summed so far
        const float alpha = __builtin_amdgcn_exp2f(fmaf(m_run[rt], a.scale_log2, -mc));  // 0 while nothing was seen
        l_run[rt] *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[rt][dt] *= alpha;
        m_run[rt] = m_new;
      }
      float psum = 0.f;
      bf16x8_t pb;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(fmaf(sc[e], a.scale_log2, -mc));
        psum += p;
        pb[e] = (__bf16)p;
      }
      l_run[rt] += psum;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        acc[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.vv[dt].whole, pb, acc[rt][dt], 0, 0, 0);
    }
  };

  StepRegs<DT> ring[PF];
  // With two row tiles (prompts: many steps a wavefront) the pages of a step are looked up when
  // the loads of the step before are issued; with one (decode: few steps) right before its own.
  constexpr bool AHEAD = BIG && RT == 2;
  StepPages pages = {};
  if (AHEAD && k_begin < k_end) pages = step_pages(a, table, k_begin, t.lo, t.hi);
  auto issue = [&](StepRegs<DT>& regs, int k) {
    if (BIG && !AHEAD) pages = step_pages(a, table, k, t.lo, t.hi);
    load_step<DT, BIG>(regs, a, table, pages, kvh, k, t.lo, t.hi, r, q);
    if (AHEAD && k + 32 < k_end) pages = step_pages(a, table, k + 32, t.lo, t.hi);
  };
#pragma unroll
  for (int i = 0; i < PF; ++i)
    if (k_begin + 32 * i < k_end) issue(ring[i], k_begin + 32 * i);
  for (int kb = k_begin; kb < k_end; kb += 32 * PF) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int k = kb + 32 * i;
      if (k < k_end) {
        compute_step(ring[i], k);
        if (k + 32 * PF < k_end) issue(ring[i], k + 32 * PF);
      }
    }
  }

  // acc[rt][dt][j] of lane (r, q) is O^T[d = 16 dt + 4q + j][row r]
  const size_t item0 = ((size_t)tile * a.nkv + kvh) * a.max_splits;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float l = l_run[rt];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    l_run[rt] = l;
    m_run[rt] *= a.scale_log2;  // from here on in units of log 2, as the merges take it
  }
  if (NW > 1) {
    // every wavefront leaves (max, sum, weighted values) of its rows; wavefront 0 adds them in order
    constexpr int ROW = D + 4;  // max, sum, two unused, then the values (16-byte aligned)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float* row = wg_part + ((size_t)wave * 16 * RT + rt * 16 + r) * ROW;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *(f32x4_t*)(row + 4 + dt * 16 + q * 4) = acc[rt][dt];
      if (q == 0) {
        row[0] = m_run[rt];
        row[1] = l_run[rt];
      }
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float m = -INFINITY;
      for (int w = 0; w < NW; ++w) m = fmaxf(m, wg_part[((size_t)w * 16 * RT + rt * 16 + r) * ROW]);
      float l = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[rt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      for (int w = 0; w < NW; ++w) {
        const float* row = wg_part + ((size_t)w * 16 * RT + rt * 16 + r) * ROW;
        const float mw = row[0];
        const float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - m);
        l += f * row[1];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[rt][dt] += f * *(const f32x4_t*)(row + 4 + dt * 16 + q * 4);
      }
      m_run[rt] = m;
      l_run[rt] = l;
    }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float l = l_run[rt];
    const int flat = flat_r[rt];
    if (flat < 0) continue;
    if (nsp == 1) {
      const int tok = flat / a.group, g = flat - tok * a.group;
      bf16_t* op = a.out + (size_t)(t.qs + tok) * a.out_stride + (size_t)(kvh * a.group + g) * D;
      const float inv = 1.0f / l;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        union { bf16_t h[4]; uint2 u; } pk;
#pragma unroll
        for (int j = 0; j < 4; ++j) pk.h[j] = __float2bfloat16(acc[rt][dt][j] * inv);
        *(uint2*)(op + dt * 16 + q * 4) = pk.u;
      }
    } else {
      const size_t item = item0 + (s - t.s_first);
      float* po = a.part_o + (item * (16 * RT) + rt * 16 + r) * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *(f32x4_t*)(po + dt * 16 + q * 4) = acc[rt][dt];
      if (q == 0) {
        float* pm = a.part_ml + (item * (16 * RT) + rt * 16 + r) * 2;
        pm[0] = m_run[rt];
        pm[1] = l;
      }
    }
  }
}

// Adds the partial results of split tiles, always in split order.  One wavefront
// per (tile, kv head, row): lane i takes the statistics of split i (of splits i, i + 64, ..),
// then every lane sums one (or more) of the row's d outputs over the splits, with the
// weights handed from lane to lane.  Where the partial results lie depends on the launch
// alone, so the first MG_AHEAD splits are loaded before the tile's range (which says how
// many of them count) has arrived: the kernel is little more than one trip to memory.
#define MG_AHEAD 16
__global__ __launch_bounds__(256) void attention_merge_kernel(AttnArgs a, int D, int row_tiles) {
  const int tile = blockIdx.x, kvh = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.z * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int rows_per_tile = 16 * row_tiles;
  const size_t item0 = ((size_t)tile * a.nkv + kvh) * a.max_splits;
  const float* ml = a.part_ml + (item0 * rows_per_tile + row) * 2;  // split sp is sp * rows_per_tile * 2 further
  const size_t ml_step = (size_t)rows_per_tile * 2;
  const float* po = a.part_o + (item0 * rows_per_tile + row) * D;
  const size_t po_step = (size_t)rows_per_tile * D;
  // ahead of everything: what may be stale or never written is not used below
  float ahead[MG_AHEAD];
  const int d_first = min(lane, D - 1);
#pragma unroll
  for (int sp = 0; sp < MG_AHEAD; ++sp) ahead[sp] = sp < a.max_splits ? po[sp * po_step + d_first] : 0.f;
  float ms_own = -INFINITY, ls_own = 0.f;
  if (lane < a.max_splits) {
    ms_own = ml[lane * ml_step];
    ls_own = ml[lane * ml_step + 1];
  }

  const TileRange t = tile_range(a, tile, row_tiles);
  const int nsp = t.s_last - t.s_first + 1;
  if (nsp == 1) return;
  const int base = row < 16 ? t.row0[0] : t.row0[1];
  const int flat = base + (row & 15);
  if (base < 0 || flat >= t.n_rows) return;
  const int tok = flat / a.group, g = flat - tok * a.group;
  bf16_t* op = a.out + (size_t)(t.qs + tok) * a.out_stride + (size_t)(kvh * a.group + g) * D;
  if (lane >= nsp) ms_own = -INFINITY;
  float m = ms_own;
  for (int sp = lane + 64; sp < nsp; sp += 64) m = fmaxf(m, ml[sp * ml_step]);
  m = wave_max(m);
  if (nsp <= 64) {
    const float w = ms_own == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms_own - m);
    const float inv = 1.0f / wave_sum(lane < nsp ? w * ls_own : 0.f);
    for (int d0 = 0; d0 < D; d0 += 64) {  // every lane stays in the loop: the weights come from all of them
      const int d = min(d0 + lane, D - 1);
      float o = 0.f;
#pragma unroll
      for (int sp = 0; sp < MG_AHEAD; ++sp) {
        const float ws = __shfl(w, sp, 64);
        const float v = d0 == 0 ? ahead[sp] : (sp < nsp ? po[sp * po_step + d] : 0.f);
        if (sp < nsp) o += ws * v;
      }
#pragma unroll 8
      for (int sp = MG_AHEAD; sp < nsp; ++sp) o += __shfl(w, sp, 64) * po[sp * po_step + d];
      if (d0 + lane < D) op[d] = __float2bfloat16(o * inv);
    }
    return;
  }
  float l = 0.f;
  for (int sp = lane; sp < nsp; sp += 64) {
    const float ms = ml[sp * ml_step];
    l += (ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - m)) * ml[sp * ml_step + 1];
  }
  const float inv = 1.0f / wave_sum(l);
  for (int d = lane; d < D; d += 64) {
    float o = 0.f;
#pragma unroll 8
    for (int sp = 0; sp < nsp; ++sp) {
      const float ms = ml[sp * ml_step];
      const float w = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - m);
      o += w * po[sp * po_step + d];
    }
    op[d] = __float2bfloat16(o * inv);
  }
}

template <int DT, int RT>
static bool launch_attn(const AttnArgs& a, int grid_splits, int nw, hipStream_t stream) {
  const size_t lds = nw > 1 ? (size_t)nw * 16 * RT * (DT * 16 + 4) * sizeof(float) : 0;
  auto kernel = a.P >= 16 ? paged_attention_mfma_kernel<DT, RT, true> : paged_attention_mfma_kernel<DT, RT, false>;
  if (lds > 64 * 1024 &&
      hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return false;
  hipLaunchKernelGGL(kernel, dim3(a.n_tiles * a.nkv, 1, grid_splits), dim3(64 * nw), lds, stream, a);
  return true;
}

template <int RT>
static bool launch_attn_d(const AttnArgs& a, int dt, int grid_splits, int nw, hipStream_t stream) {
  switch (dt) {
    case 1: return launch_attn<1, RT>(a, grid_splits, nw, stream);
    case 2: return launch_attn<2, RT>(a, grid_splits, nw, stream);
    case 3: return launch_attn<3, RT>(a, grid_splits, nw, stream);
    case 4: return launch_attn<4, RT>(a, grid_splits, nw, stream);
    case 5: return launch_attn<5, RT>(a, grid_splits, nw, stream);
    case 6: return launch_attn<6, RT>(a, grid_splits, nw, stream);
    case 7: return launch_attn<7, RT>(a, grid_splits, nw, stream);
    case 8: return launch_attn<8, RT>(a, grid_splits, nw, stream);
    default: return false;
  }
}

// A wavefront owns row_tiles (1 or 2) tiles of 16 rows of one request: the rows from
// tile_row0[i] and, with two, the rows from tile_row1[i] (-1: none; a null tile_row1: the
// 16 rows after the first tile).  `waves` wavefronts share a split (at most 16; 8 with a
// head size above 64; 4 with two row tiles).  `grid_splits` is an upper bound on the
// splits of any tile and `max_splits` the number the scratch has room for (grid_splits <=
// max_splits).  part_o holds tiles * nkv * max_splits * 16 * row_tiles * d floats, part_ml
// tiles * nkv * max_splits * 16 * row_tiles * 2 (both may be null when max_splits is 1).
// Launches that share scratch must not overlap.
TK_API int tk_paged_attention_mfma(const void* q, int q_stride, void* out, int out_stride,
                                       const void* kcache, const void* vcache,
                                       const int* block_table, int table_stride,
                                       const int* q_start, const int* kv_len,
                                       const int* tile_req, const int* tile_row0, const int* tile_row1,
                                       int n_tiles, int row_tiles, int nq, int nkv, int d, int P, int window,
                                       float scale, int split, int waves, int grid_splits, int max_splits,
                                       float* part_o, float* part_ml, hipStream_t stream) {
  TK_REQUIRE(n_tiles >= 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention_mfma: bad sizes tiles=%d nq=%d nkv=%d", n_tiles, nq, nkv);
  TK_REQUIRE(d % 16 == 0 && d >= 16 && d <= 128, "attention_mfma: head size %d is not a multiple of 16 up to 128", d);
  TK_REQUIRE(P >= 4 && (P & (P - 1)) == 0, "attention_mfma: page size %d is not a power of two from 4", P);
  TK_REQUIRE(scale > 0.f, "attention_mfma: the scale must be positive");
  TK_REQUIRE(row_tiles == 1 || row_tiles == 2, "attention_mfma: row_tiles %d outside 1..2", row_tiles);
  TK_REQUIRE(row_tiles == 2 || !tile_row1, "attention_mfma: second row tiles given with one row tile a wavefront");
  TK_REQUIRE(split > 0 && split % 32 == 0, "attention_mfma: split %d is not a multiple of 32", split);
  TK_REQUIRE(waves >= 1 && waves <= max_waves(d / 16, row_tiles) && split % (32 * waves) == 0,
             "attention_mfma: %d wavefronts (at most %d) do not cut a split of %d keys into multiples of 32", waves,
             max_waves(d / 16, row_tiles), split);
  TK_REQUIRE((size_t)waves * 16 * row_tiles * (d + 4) * sizeof(float) <= 160 * 1024 || waves == 1,
             "attention_mfma: %d wavefronts of head size %d do not fit the local memory", waves, d);
  TK_REQUIRE(grid_splits >= 1 && grid_splits <= max_splits && grid_splits < 65536, "attention_mfma: splits %d of %d", grid_splits, max_splits);
  TK_REQUIRE(max_splits == 1 || (part_o && part_ml), "attention_mfma: split tiles need scratch");
  TK_REQUIRE(q_stride >= nq * d && out_stride >= nq * d && q_stride % 8 == 0 && out_stride % 4 == 0,
             "attention_mfma: row strides %d/%d too short or unaligned", q_stride, out_stride);
  TK_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 7) == 0 && ((uintptr_t)out & 7) == 0,
             "attention_mfma: operands must be 16-byte aligned");
  TK_REQUIRE(nkv < 65536, "attention_mfma: too many kv heads");
  if (n_tiles == 0) return 0;
  AttnArgs a;
  a.q = (const bf16_t*)q; a.q_stride = q_stride; a.out = (bf16_t*)out; a.out_stride = out_stride;
  a.kcache = (const bf16_t*)kcache; a.vcache = (const bf16_t*)vcache;
  a.block_table = block_table; a.table_stride = table_stride; a.q_start = q_start; a.kv_len = kv_len;
  a.tile_req = tile_req; a.tile_row0 = tile_row0; a.tile_row1 = tile_row1; a.n_tiles = n_tiles;
  a.nq = nq; a.nkv = nkv; a.group = nq / nkv; a.P = P; a.window = window;
  a.p_shift = 0;
  while ((1 << a.p_shift) < P) ++a.p_shift;
  a.scale_log2 = scale * 1.4426950408889634f;
  a.split = split; a.max_splits = max_splits; a.part_o = part_o; a.part_ml = part_ml;
  const bool ok = row_tiles == 1 ? launch_attn_d<1>(a, d / 16, grid_splits, waves, stream)
                                 : launch_attn_d<2>(a, d / 16, grid_splits, waves, stream);
  TK_REQUIRE(ok, "attention_mfma: no kernel for head size %d", d);
  TK_CHECK_LAUNCH("paged_attention_mfma");
  if (max_splits > 1) {
    const int rows = 16 * row_tiles;
    hipLaunchKernelGGL(attention_merge_kernel, dim3(n_tiles, nkv, rows / 4), dim3(256), 0, stream, a, d, row_tiles);
    TK_CHECK_LAUNCH("attention_merge");
  }
  return 0;
}
