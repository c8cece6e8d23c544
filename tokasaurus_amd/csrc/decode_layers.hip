// A run of transformer blocks for a decode step of few tokens (one token a request, at most
// 16 requests) in ONE kernel: per block  RMSNorm -> q|k|v product -> rotation, append to the
// pages -> attention over the pages -> output product + residual -> RMSNorm -> gate|up product,
// SwiGLU -> down product + residual.
//
// Why one kernel.  Launched one by one, the six kernels of a block each cost a round of
// workgroups that ramps up, waits a trip to memory and drains: 4 to 9 us for products whose
// bytes need 1 to 8 us, 97 times a step.  Here one workgroup per compute unit stays resident
// for the whole run; the phases of a block are separated by barriers across the grid (about
// 2 us each), and a phase's weights are streamed by the same wavefronts that will multiply them.
//
// Work of a phase.  A product phase cuts the output rows (for q|k|v the pairs of rows that
// the rotation joins, for gate|up the pairs (gate row, up row)) evenly over the workgroups; a
// workgroup's 8 wavefronts split K, every wavefront streams its part of the workgroup's weight
// rows through v_mfma_f32_16x16x32_bf16 (weight tile first operand, the tokens second), and the
// partial sums meet in LDS in wavefront order, so every output has one order of summation.
// The attention phase gives each (request, kv head, split of the keys) to a workgroup whose
// wavefronts split the keys again (attention_mfma.h); the partial results of the splits are
// merged, in split order, by the output product's wavefronts as they build their operand.
//
// Data between workgroups (the residual stream, q, the attention's partial results, the
// gate|up result, the new key and value in the pages) is written with stores that write
// through the caches and read with loads that go around them (agent-scope relaxed atomics),
// because each of the chip's eight dies has an L2 of its own; the grid barrier then needs no
// cache-wide write-back or invalidation, only a wait for the workgroup's own stores.
//
// The grid barrier: workgroups arrive at a counter of their group of 16, the last of a group
// at the top counter, the last there raises every group's flag, which the group's workgroups
// poll.  Counters only grow (the round number carries over from launch to launch in the sync
// words), so nothing has to be cleared between launches.  Every wait is bounded: after
// `spin_cap` polls a workgroup gives up, sets the status word, skips every later barrier and
// runs to the end, so every workgroup always exits; the host finds the status word set and
// raises an error.  All workgroups must be resident together: the grid is at most the number of
// compute units and a workgroup takes a compute unit's worth of wavefront slots or LDS.
#include "attention_mfma.h"

#define DL_WAVES 8            // wavefronts of a workgroup
#define DL_THREADS (64 * DL_WAVES)
#define DL_RING 8             // (tile, step) slots whose loads a wavefront keeps in flight
#define DL_MAX_TILES 4        // 16-row tiles (or tile pairs) a workgroup may own in one phase
#define DL_FAN 16             // workgroups per first-level counter of the barrier
#define DL_MAX_GROUPS 4096    // workgroups a launch may have
#define DL_MAX_TABLES 4       // block tables (cache groups) a run of blocks may use

// words of the sync buffer (uint32), 16 apart so that each sits in a cache line of its own
#define DL_SYNC_GROUP(g) (16 * (g))
#define DL_SYNC_TOP (16 * (DL_MAX_GROUPS / DL_FAN))
#define DL_SYNC_FLAG(g) (16 * (DL_MAX_GROUPS / DL_FAN + 1 + (g)))
#define DL_SYNC_EPOCH (16 * (2 * (DL_MAX_GROUPS / DL_FAN) + 1))
#define DL_SYNC_WORDS (16 * (2 * (DL_MAX_GROUPS / DL_FAN) + 2))

// One block of the run, in device memory (written once by the host when the model is set up).
struct DecodeLayer {
  const bf16_t* w_qkv;   // [(nq + 2 nkv) d, H]
  const bf16_t* w_o;     // [H, nq d]
  const bf16_t* w_gu;    // [2 I, H], gate rows then up rows
  const bf16_t* w_down;  // [H, I]
  const void* norm1;     // [H] weight of the norm before the mixer
  const void* norm2;     // [H] weight of the norm before the feed-forward
  bf16_t* kcache;        // this block's pages of keys
  bf16_t* vcache;
  const float* cos_t;    // [positions][d / 2], null: no rotation
  const float* sin_t;
  float eps1, eps2;
  int norm1_f32, norm2_f32;  // the norm weights are 32-bit
  int window;                // 0: every key
  int table;                 // which of the step's block tables this block's cache uses
};

struct DecodeArgs {
  const DecodeLayer* layers;
  int n_layers;
  int M, H, I, nq, nkv, d, P;
  const int* positions;  // [M]
  const int* kv_len;     // [M] keys of each request after this step's append (position + 1)
  const int* tables[DL_MAX_TABLES];  // block tables [M, stride]
  int table_stride[DL_MAX_TABLES];
  bf16_t* x;   // [M, H] the residual stream: in, and out after the last block
  bf16_t* xb;  // [M, H] scratch: the stream between mixer and feed-forward
  bf16_t* q;   // [M, nq d] scratch
  bf16_t* h;   // [M, I] scratch
  float* part_o;   // [M][nkv][max_splits][16][d] partial attention results
  float* part_ml;  // [M][nkv][max_splits][16][2]
  int split, max_splits;
  float scale;
  // for the norm that follows the run (null: none): x * w rounded once, and per row one
  // partial sum of squares a workgroup
  const void* emit_w;
  int emit_w_f32;
  bf16_t* emit_scaled;
  float* emit_sumsq;
  uint32_t* sync;    // DL_SYNC_WORDS words, zero before the first launch
  uint32_t* status;  // set to non-zero when a wait gave up
  uint32_t spin_cap;
  uint32_t expect_groups;  // workgroups the barrier waits for (the grid's size; tests pass one more)
  // diagnostics (null: none): workgroup `timing_group` writes the constant-rate clock (100 MHz)
  // at the start and, per block, after each of the 5 phases and each of the 5 barriers:
  // 1 + 10 * n_layers words
  unsigned long long* timing;
  int timing_group;
};

// ---------------------------------------------------------------------------------
// the barrier across the grid
// ---------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t sync_load(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void sync_store(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t sync_add(uint32_t* p, uint32_t v) {
  return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct GridSync {
  uint32_t* words;
  uint32_t* status;
  uint32_t round;       // rounds completed so far, over all launches
  uint32_t group, group_size, n_top;
  uint32_t spin_cap;
  bool failed;
};

__device__ __forceinline__ GridSync grid_sync_begin(const DecodeArgs& a) {
  GridSync s;
  s.words = a.sync;
  s.status = a.status;
  s.spin_cap = a.spin_cap;
  s.failed = false;
  const uint32_t groups = a.expect_groups;
  s.n_top = (groups + DL_FAN - 1) / DL_FAN;
  s.group = blockIdx.x / DL_FAN;
  s.group_size = min((uint32_t)DL_FAN, groups - s.group * DL_FAN);
  // the epoch is written by the last arrival at a launch's last barrier, after every workgroup
  // of that launch has read it here
  s.round = threadIdx.x == 0 ? sync_load(a.sync + DL_SYNC_EPOCH) : 0;
  return s;
}

// Every wavefront of every workgroup calls this.  `last`: the launch's last barrier, whose last
// arrival also stores the epoch for the next launch.
__device__ __forceinline__ void grid_barrier(GridSync& s, bool last) {
  // this wavefront's stores (write-through) are complete; then the workgroup's
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  if (threadIdx.x == 0) {
    s.round += 1;
    if (!s.failed) {
      const uint32_t round = s.round;
      const uint32_t old = sync_add(s.words + DL_SYNC_GROUP(s.group), 1u);
      if (old + 1 == round * s.group_size) {
        const uint32_t t = sync_add(s.words + DL_SYNC_TOP, 1u);
        if (t + 1 == round * s.n_top) {
          if (last) sync_store(s.words + DL_SYNC_EPOCH, round);
          for (uint32_t k = 0; k < s.n_top; ++k) sync_store(s.words + DL_SYNC_FLAG(k), round);
        }
      }
      uint32_t spins = 0;
      while ((int32_t)(sync_load(s.words + DL_SYNC_FLAG(s.group)) - round) < 0) {
        ++spins;
        if (spins > s.spin_cap || ((spins & 255u) == 0 && sync_load(s.status) != 0)) {
          s.failed = true;
          atomicOr(s.status, 1u);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// ---------------------------------------------------------------------------------
// a product phase
// ---------------------------------------------------------------------------------
__device__ __forceinline__ bf16x8_t dl_zero8() {
  bf16x8_t z;
#pragma unroll
  for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.f;
  return z;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// LDS of a product phase: [ssq: DL_WAVES x 16 floats][sums: (PAIRED ? 2 : 1) x tiles x DL_WAVES x 64 f32x4]
#define DL_SSQ_FLOATS (DL_WAVES * 16)

struct PhaseShape {
  int u0, u1, nt, th;  // this workgroup's units [u0, u1), in nt tiles of th units
};

__device__ __forceinline__ PhaseShape phase_shape(int units) {
  PhaseShape p;
  const int G = gridDim.x, g = blockIdx.x;
  const int upw = (units + G - 1) / G;
  p.u0 = min(units, g * upw);
  p.u1 = min(units, p.u0 + upw);
  p.nt = (p.u1 - p.u0 + 15) >> 4;
  p.th = p.nt ? (p.u1 - p.u0 + p.nt - 1) / p.nt : 0;
  return p;
}

// C[token][unit] = sum_k A[token][k] W[row(unit)][k] for this workgroup's units.
//   PAIRED: a unit is two rows, row(unit) and row(unit) + pair_off; `half` > 0 maps unit u to
//   row (u / half) * 2 half + u % half (the first of a rotation's pair), else row = unit.
//   load_a(step, first_pass) gives lane (token r, quarter q) its 8 values A[r][32 step + 8 q ..];
//   first_pass is true in the workgroup's first tile (statistics of A are taken there, once).
//   before_sync(): called by every wavefront after its last product, before the workgroup's
//   barrier (statistics go to LDS here).
//   epilogue(token, slot, unit0, limit, s0, s1): the sums of units unit0 .. unit0 + 3 (those
//   below `limit` exist) for one token, s1 the paired rows'; slot = tile * 4 + quarter numbers
//   the calls of one token.
template <bool PAIRED, typename LoadA, typename BeforeSync, typename Epilogue>
__device__ __forceinline__ void product_phase(const bf16_t* __restrict__ W, const int K, const int units, const int half,
                                              const int pair_off, float* lds, LoadA load_a, BeforeSync before_sync,
                                              Epilogue epilogue) {
  const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, q = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const PhaseShape p = phase_shape(units);
  const int K32 = (K + 31) >> 5;
  const int ks0 = K32 * wave / DL_WAVES, ks1 = K32 * (wave + 1) / DL_WAVES;
  const int n_steps = ks1 - ks0;
  const int n_slots = p.nt * n_steps;
  f32x4_t* red = (f32x4_t*)(lds + DL_SSQ_FLOATS);
  f32x4_t* red2 = red + p.nt * DL_WAVES * 64;

  // the weight row of this lane in a tile
  auto row_of = [&](int tile, bool& ok) -> const bf16_t* {
    const int unit = p.u0 + tile * p.th + r;
    ok = r < p.th && unit < p.u1;
    const int uu = ok ? unit : p.u0;
    const int row = half > 0 ? (uu / half) * (2 * half) + uu % half : uu;
    return W + (size_t)row * K + q * 8;
  };

  bf16x8_t wa[DL_RING], wb[DL_RING], av[DL_RING];
  int i_tile = 0, i_step = 0;
  bool ok_i = false;
  const bf16_t* p_i = p.nt > 0 ? row_of(0, ok_i) : W;
  auto issue = [&](bf16x8_t& w0, bf16x8_t& w1, bf16x8_t& a0) {
    if (i_tile < p.nt && n_steps > 0) {
      const int step = ks0 + i_step;
      const bool ok = ok_i && step * 32 + q * 8 < K;
      if (ok) {
        w0 = *(const bf16x8_t*)(p_i + (size_t)step * 32);
        if (PAIRED) w1 = *(const bf16x8_t*)(p_i + (size_t)pair_off * K + (size_t)step * 32);
      } else {
        w0 = dl_zero8();
        if (PAIRED) w1 = dl_zero8();
      }
      a0 = load_a(step, i_tile == 0);
      if (++i_step == n_steps) {
        i_step = 0;
        ++i_tile;
        if (i_tile < p.nt) p_i = row_of(i_tile, ok_i);
      }
    }
  };
#pragma unroll
  for (int j = 0; j < DL_RING; ++j) issue(wa[j], wb[j], av[j]);

  f32x4_t acc0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, acc1 = acc0;
  int c_tile = 0, c_step = 0;
  for (int base = 0; base < n_slots; base += DL_RING) {
#pragma unroll
    for (int j = 0; j < DL_RING; ++j) {
      if (base + j < n_slots) {
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[j], av[j], acc0, 0, 0, 0);
        if (PAIRED) acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[j], av[j], acc1, 0, 0, 0);
        if (++c_step == n_steps) {
          red[(c_tile * DL_WAVES + wave) * 64 + lane] = acc0;
          if (PAIRED) red2[(c_tile * DL_WAVES + wave) * 64 + lane] = acc1;
          acc0 = f32x4_t{0.f, 0.f, 0.f, 0.f};
          acc1 = acc0;
          c_step = 0;
          ++c_tile;
        }
        issue(wa[j], wb[j], av[j]);
      }
    }
  }
  if (n_steps == 0) {
    // a wavefront without a part of K still owes its (zero) sums
    for (int t = 0; t < p.nt; ++t) {
      red[(t * DL_WAVES + wave) * 64 + lane] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (PAIRED) red2[(t * DL_WAVES + wave) * 64 + lane] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  }
  before_sync();
  __syncthreads();
  for (int u = tid; u < p.nt * 64; u += DL_THREADS) {
    const int l = u & 63, t = u >> 6;
    f32x4_t s0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
    for (int w = 0; w < DL_WAVES; ++w) {
      s0 += red[(t * DL_WAVES + w) * 64 + l];
      if (PAIRED) s1 += red2[(t * DL_WAVES + w) * 64 + l];
    }
    const int unit0 = p.u0 + t * p.th + (l >> 4) * 4;
    const int limit = min(p.u1, p.u0 + (t + 1) * p.th);
    epilogue(l & 15, t * 4 + (l >> 4), unit0, limit, s0, s1);
  }
}

// lane (token r, quarter q): 8 values of a [M, K] bfloat16 matrix written by other workgroups
__device__ __forceinline__ bf16x8_t load_rows(const bf16_t* A, int lda, int M, int K, int step, int r, int q) {
  const int k0 = step * 32 + q * 8;
  if (r >= M || k0 >= K) return dl_zero8();
  return load_bf16x8<true>(A + (size_t)r * lda + k0);
}

// The operand of a product behind an RMSNorm: x * w rounded once (the rows are divided by their
// rms after the product), and the sum of x^2 over what this lane saw.
__device__ __forceinline__ bf16x8_t load_normed(const bf16_t* x, int H, int M, const void* w, int w_f32, int step, int r,
                                                int q, bool first, float& ssq) {
  const int k0 = step * 32 + q * 8;
  if (r >= M || k0 >= H) return dl_zero8();
  union { uint64_t u[2]; uint16_t h[8]; } xv;
  xv.u[0] = shared_load64(x + (size_t)r * H + k0);
  xv.u[1] = shared_load64(x + (size_t)r * H + k0 + 4);
  float wv[8];
  if (w_f32) {
    const f32x4_t a = *(const f32x4_t*)((const float*)w + k0), b = *(const f32x4_t*)((const float*)w + k0 + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { wv[e] = a[e]; wv[4 + e] = b[e]; }
  } else {
    union { uint4 u; uint16_t h[8]; } ww;
    ww.u = *(const uint4*)((const bf16_t*)w + k0);
#pragma unroll
    for (int e = 0; e < 8; ++e) wv[e] = bf16_bits_to_f32(ww.h[e]);
  }
  bf16x8_t out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float xr = bf16_bits_to_f32(xv.h[e]);
    if (first) ssq = fmaf(xr, xr, ssq);
    out[e] = (__bf16)(wv[e] * xr);
  }
  return out;
}

// This wavefront's sums of squares, one a token, to LDS; after the workgroup's barrier
// rstd_of() adds the wavefronts' parts in wavefront order.
__device__ __forceinline__ void put_ssq(float* lds, float ssq, int wave, int lane) {
  ssq += __shfl_xor(ssq, 16, 64);
  ssq += __shfl_xor(ssq, 32, 64);
  if (lane < 16) lds[wave * 16 + lane] = ssq;
}
__device__ __forceinline__ float rstd_of(const float* lds, int token, int K, float eps) {
  float ss = 0.f;
#pragma unroll
  for (int w = 0; w < DL_WAVES; ++w) ss += lds[w * 16 + token];
  return 1.0f / sqrtf(ss / (float)K + eps);
}

__device__ __forceinline__ uint16_t bf16_bits(float v) {
  union { bf16_t h; uint16_t u; } x;
  x.h = __float2bfloat16(v);
  return x.u;
}

// four outputs of one token to a bfloat16 row that other workgroups read
__device__ __forceinline__ void store_row4(bf16_t* row, int n, int limit, const float (&o)[4]) {
  if (n + 3 < limit && (n & 3) == 0 && (((uintptr_t)row) & 7) == 0) {
    union { uint64_t u; uint16_t h[4]; } pk;
#pragma unroll
    for (int j = 0; j < 4; ++j) pk.h[j] = bf16_bits(o[j]);
    shared_store64(row + n, pk.u);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < limit) shared_store16(row + n + j, bf16_bits(o[j]));
  }
}

// ---------------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------------
template <int DT, bool BIG>
__global__ __launch_bounds__(DL_THREADS) void decode_layers_kernel(DecodeArgs a) {
  extern __shared__ __align__(16) float lds[];
  constexpr int D = DT * 16;
  const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, q = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int M = a.M, H = a.H, I = a.I, nq = a.nq, nkv = a.nkv, P = a.P;
  const int half = D / 2, group = nq / nkv;
  GridSync gs = grid_sync_begin(a);
  const bool timed = a.timing != nullptr && (int)blockIdx.x == a.timing_group && tid == 0;
  if (timed) a.timing[0] = wall_clock64();
  int mark_at = 1;
  auto mark = [&]() {
    if (timed) a.timing[mark_at] = wall_clock64();
    ++mark_at;
  };

  for (int li = 0; li < a.n_layers; ++li) {
    const DecodeLayer L = a.layers[li];
    const int* table = a.tables[L.table];
    const int table_stride = a.table_stride[L.table];
    const bool last_layer = li + 1 == a.n_layers;

    // ---- 1. q | k | v of the normed stream, rotated; q to scratch, k and v to the pages
    {
      float ssq = 0.f;
      product_phase<true>(
          L.w_qkv, H, (nq + 2 * nkv) * half, half, half, lds,
          [&](int step, bool first) { return load_normed(a.x, H, M, L.norm1, L.norm1_f32, step, r, q, first, ssq); },
          [&]() { put_ssq(lds, ssq, wave, lane); },
          [&](int token, int, int unit0, int limit, f32x4_t s0, f32x4_t s1) {
            if (token >= M) return;
            const float rstd = rstd_of(lds, token, H, L.eps1);
            const int pos = a.positions[token];
            const int page = table[(size_t)token * table_stride + pos / P];
            const int off = pos % P;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int unit = unit0 + j;
              if (unit >= limit) continue;
              const int head = unit / half, c = unit - head * half;
              const float x1 = round_to<bf16_t>(s0[j] * rstd), x2 = round_to<bf16_t>(s1[j] * rstd);
              float o1 = x1, o2 = x2;
              if (head < nq + nkv && L.cos_t != nullptr)
                rotate_pair(x1, x2, L.cos_t[(size_t)pos * half + c], L.sin_t[(size_t)pos * half + c], o1, o2);
              if (head < nq) {
                bf16_t* dst = a.q + (size_t)token * (nq * D) + (size_t)head * D + c;
                shared_store16(dst, bf16_bits(o1));
                shared_store16(dst + half, bf16_bits(o2));
              } else if (head < nq + nkv) {
                bf16_t* dst = L.kcache + ((size_t)page * nkv + (head - nq)) * P * D;
                shared_store16(dst + key_offset(P, off, c), bf16_bits(o1));
                shared_store16(dst + key_offset(P, off, c + half), bf16_bits(o2));
              } else {
                bf16_t* dst = L.vcache + ((size_t)page * nkv + (head - nq - nkv)) * P * D;
                shared_store16(dst + value_offset(D, off, c), bf16_bits(o1));
                shared_store16(dst + value_offset(D, off, c + half), bf16_bits(o2));
              }
            }
          });
    }
    mark();
    grid_barrier(gs, false);
    mark();

    // ---- 2. attention of every (request, kv head) over its pages, the keys cut into splits
    {
      AttnArgs at;
      at.q = a.q; at.q_stride = nq * D; at.out = nullptr; at.out_stride = 0;
      at.kcache = L.kcache; at.vcache = L.vcache;
      at.block_table = table; at.table_stride = table_stride;
      at.q_start = nullptr; at.kv_len = a.kv_len; at.tile_req = nullptr; at.tile_row0 = nullptr; at.tile_row1 = nullptr;
      at.n_tiles = M; at.nq = nq; at.nkv = nkv; at.group = group; at.P = P; at.window = L.window;
      at.p_shift = 31 - __builtin_clz(P);
      at.scale_log2 = a.scale * 1.4426950408889634f;
      at.split = a.split; at.max_splits = a.max_splits; at.part_o = a.part_o; at.part_ml = a.part_ml;
      const int n_items = M * nkv * a.max_splits;
      for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int split_index = item % a.max_splits, rest = item / a.max_splits;
        attention_item<DT, 1, BIG, true>(at, rest / nkv, rest % nkv, split_index, lds, DL_WAVES);
        __syncthreads();  // the next item uses the same LDS
      }
    }
    mark();
    grid_barrier(gs, false);
    mark();

    // ---- 3. xb = x + attention * Wo^T; the attention's splits are merged on the way in
    product_phase<false>(
        L.w_o, nq * D, H, 0, 0, lds,
        [&](int step, bool) -> bf16x8_t {
          const int k0 = step * 32 + q * 8;
          if (r >= M || k0 >= nq * D) return dl_zero8();
          const int head = k0 / D, c0 = k0 - head * D;
          const int kvh = head / group, row = head - kvh * group;
          const int kvl = a.kv_len[r];
          const int lo = L.window > 0 ? max(0, kvl - L.window) : 0;
          const int s_first = lo / a.split, nsp = (kvl - 1) / a.split - s_first + 1;
          const size_t item0 = ((size_t)r * nkv + kvh) * a.max_splits;
          const float* ml = a.part_ml + (item0 * 16 + row) * 2;
          const float* po = a.part_o + (item0 * 16 + row) * D + c0;
          float m = -INFINITY;
          for (int sp = 0; sp < nsp; ++sp) {
            union { uint64_t u; float f[2]; } v;
            v.u = shared_load64(ml + (size_t)sp * 32);
            m = fmaxf(m, v.f[0]);
          }
          float l = 0.f, o[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = 0.f;
          for (int sp = 0; sp < nsp; ++sp) {
            union { uint64_t u; float f[2]; } v;
            v.u = shared_load64(ml + (size_t)sp * 32);
            const float w = v.f[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(v.f[0] - m);
            l += w * v.f[1];
            const float* src = po + (size_t)sp * 16 * D;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
              union { uint64_t u; float f[2]; } pv;
              pv.u = shared_load64(src + e);
              o[e] += w * pv.f[0];
              o[e + 1] += w * pv.f[1];
            }
          }
          const float inv = 1.0f / l;
          bf16x8_t out;
#pragma unroll
          for (int e = 0; e < 8; ++e) out[e] = (__bf16)(o[e] * inv);
          return out;
        },
        [&]() {},
        [&](int token, int, int unit0, int limit, f32x4_t s0, f32x4_t) {
          if (token >= M) return;
          float o[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            o[j] = 0.f;
            if (unit0 + j < limit) {
              union { uint16_t u; } res;
              // the residual is this workgroup's own slice of x, but written by another phase's workgroups
              res.u = __hip_atomic_load((const uint16_t*)(a.x + (size_t)token * H + unit0 + j), __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
              o[j] = round_to<bf16_t>(s0[j]) + bf16_bits_to_f32(res.u);
            }
          }
          store_row4(a.xb + (size_t)token * H, unit0, limit, o);
        });
    mark();
    grid_barrier(gs, false);
    mark();

    // ---- 4. h = silu(gate) * up of the normed stream
    {
      float ssq = 0.f;
      product_phase<true>(
          L.w_gu, H, I, 0, I, lds,
          [&](int step, bool first) { return load_normed(a.xb, H, M, L.norm2, L.norm2_f32, step, r, q, first, ssq); },
          [&]() { put_ssq(lds, ssq, wave, lane); },
          [&](int token, int, int unit0, int limit, f32x4_t s0, f32x4_t s1) {
            if (token >= M) return;
            const float rstd = rstd_of(lds, token, H, L.eps2);
            float o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = silu_mul_bf16(s0[j] * rstd, s1[j] * rstd);
            store_row4(a.h + (size_t)token * I, unit0, limit, o);
          });
    }
    mark();
    grid_barrier(gs, false);
    mark();

    // ---- 5. x = xb + h * Wdown^T (and, after the last block, what the following norm needs)
    {
      float* emit_part = lds + DL_SSQ_FLOATS + DL_MAX_TILES * DL_WAVES * 64 * 4;  // [tile * 4 + quarter][16 tokens], behind the sums
      const bool emit = last_layer && a.emit_w != nullptr;
      const PhaseShape shape = phase_shape(H);
      product_phase<false>(
          L.w_down, I, H, 0, 0, lds,
          [&](int step, bool) { return load_rows(a.h, I, M, I, step, r, q); },
          [&]() {},
          [&](int token, int slot, int unit0, int limit, f32x4_t s0, f32x4_t) {
            float o[4], ss = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              o[j] = 0.f;
              if (token < M && unit0 + j < limit) {
                const uint16_t res = __hip_atomic_load((const uint16_t*)(a.xb + (size_t)token * H + unit0 + j),
                                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                o[j] = round_to<bf16_t>(s0[j]) + bf16_bits_to_f32(res);
              }
            }
            if (token < M) store_row4(a.x + (size_t)token * H, unit0, limit, o);
            if (emit) {
              float sc[4];
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                sc[j] = 0.f;
                if (token < M && unit0 + j < limit) {
                  const float xr = round_to<bf16_t>(o[j]);
                  const float w = a.emit_w_f32 ? ((const float*)a.emit_w)[unit0 + j]
                                               : __bfloat162float(((const bf16_t*)a.emit_w)[unit0 + j]);
                  ss = fmaf(xr, xr, ss);
                  sc[j] = w * xr;
                }
              }
              if (token < M) store_row4(a.emit_scaled + (size_t)token * H, unit0, limit, sc);
              emit_part[slot * 16 + token] = ss;  // (tile, quarter, token): a place of its own
            }
          });
      if (emit) {
        __syncthreads();
        if (tid < M) {
          float ss = 0.f;
          for (int k = 0; k < shape.nt * 4; ++k) ss += emit_part[k * 16 + tid];
          union { float f; uint32_t u; } v;
          v.f = ss;
          __hip_atomic_store((uint32_t*)(a.emit_sumsq + (size_t)tid * gridDim.x + blockIdx.x), v.u, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    mark();
    grid_barrier(gs, last_layer);
    mark();
  }
}

// ---------------------------------------------------------------------------------
// launch
// ---------------------------------------------------------------------------------
static size_t decode_lds_bytes(int d) {
  const size_t product = sizeof(float) * (DL_SSQ_FLOATS + (size_t)2 * DL_MAX_TILES * DL_WAVES * 64 * 4);
  const size_t emit = sizeof(float) * (DL_SSQ_FLOATS + (size_t)DL_MAX_TILES * DL_WAVES * 64 * 4 + DL_MAX_TILES * 4 * 16);
  const size_t attention = sizeof(float) * (size_t)DL_WAVES * 16 * (d + 4);
  size_t n = product > emit ? product : emit;
  return n > attention ? n : attention;
}

static int decode_groups() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    return 0;
  return n < DL_MAX_GROUPS ? n : DL_MAX_GROUPS;
}

template <int DT>
static bool launch_decode(const DecodeArgs& a, int groups, hipStream_t stream) {
  const size_t lds = decode_lds_bytes(DT * 16);
  auto kernel = a.P >= 16 ? decode_layers_kernel<DT, true> : decode_layers_kernel<DT, false>;
  if (lds > 64 * 1024 &&
      hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return false;
  hipLaunchKernelGGL(kernel, dim3(groups), dim3(DL_THREADS), lds, stream, a);
  return true;
}

// Words the sync buffer must have (uint32, zeroed once) and workgroups a launch will use on the
// current device (0: the device could not be asked).
TK_API int tk_decode_layers_sync_words() { return DL_SYNC_WORDS; }
TK_API int tk_decode_layers_groups() { return decode_groups(); }
TK_API int tk_decode_layers_layer_bytes() { return (int)sizeof(DecodeLayer); }

// Whether the kernel takes these sizes (0), or why not (-1 and tk_last_error).
static int decode_check(int M, int H, int I, int nq, int nkv, int d, int P, int groups) {
  TK_REQUIRE(M >= 1 && M <= 16, "decode_layers: %d tokens, the kernel takes 1 to 16", M);
  TK_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0 && nq / nkv <= 16,
             "decode_layers: %d query heads over %d kv heads (at most 16 a kv head)", nq, nkv);
  TK_REQUIRE(d % 16 == 0 && d >= 16 && d <= 128, "decode_layers: head size %d is not a multiple of 16 up to 128", d);
  TK_REQUIRE(P >= 4 && (P & (P - 1)) == 0, "decode_layers: page size %d is not a power of two from 4", P);
  TK_REQUIRE(H > 0 && I > 0 && H % 8 == 0 && I % 8 == 0, "decode_layers: widths %d and %d must be multiples of 8", H, I);
  TK_REQUIRE(groups >= 1 && groups <= DL_MAX_GROUPS, "decode_layers: %d workgroups", groups);
  const int limit = 16 * DL_MAX_TILES;
  const int units[4] = {(nq + 2 * nkv) * (d / 2), H, I, H};
  for (int i = 0; i < 4; ++i)
    TK_REQUIRE((units[i] + groups - 1) / groups <= limit,
               "decode_layers: %d outputs over %d workgroups are more than %d each", units[i], groups, limit);
  return 0;
}

TK_API int tk_decode_layers_supports(int M, int H, int I, int nq, int nkv, int d, int P) {
  const int groups = decode_groups();
  TK_REQUIRE(groups > 0, "decode_layers: the device's compute units could not be counted");
  return decode_check(M, H, I, nq, nkv, d, P, groups);
}

// Runs the blocks of `args->layers` on the M rows of args->x.  The sync words carry the barrier's
// round from launch to launch: launches that share them must not overlap, and after a launch
// that set the status word both must be zeroed before the next.  groups: 0 = one workgroup a
// compute unit.
TK_API int tk_decode_layers(const DecodeArgs* args, int groups, hipStream_t stream) {
  TK_REQUIRE(args != nullptr, "decode_layers: no arguments");
  DecodeArgs a = *args;
  if (groups <= 0) groups = decode_groups();
  TK_REQUIRE(groups > 0, "decode_layers: the device's compute units could not be counted");
  if (decode_check(a.M, a.H, a.I, a.nq, a.nkv, a.d, a.P, groups) != 0) return -1;
  TK_REQUIRE(a.n_layers >= 0 && (a.n_layers == 0 || a.layers != nullptr), "decode_layers: no layers");
  TK_REQUIRE(a.positions && a.kv_len && a.x && a.xb && a.q && a.h && a.part_o && a.part_ml && a.sync && a.status,
             "decode_layers: an operand is missing");
  TK_REQUIRE(a.split > 0 && a.split % (32 * DL_WAVES) == 0 && a.max_splits >= 1,
             "decode_layers: a split of %d keys is no multiple of %d", a.split, 32 * DL_WAVES);
  TK_REQUIRE(a.scale > 0.f, "decode_layers: the scale must be positive");
  TK_REQUIRE((((uintptr_t)a.x | (uintptr_t)a.xb | (uintptr_t)a.q | (uintptr_t)a.h | (uintptr_t)a.part_o |
               (uintptr_t)a.part_ml) & 15) == 0, "decode_layers: operands must be 16-byte aligned");
  TK_REQUIRE(a.emit_w == nullptr || (a.emit_scaled && a.emit_sumsq), "decode_layers: outputs for the following norm are missing");
  TK_REQUIRE(a.spin_cap > 0, "decode_layers: the spin limit must be positive");
  if (a.expect_groups == 0) a.expect_groups = (uint32_t)groups;
  if (a.n_layers == 0) return 0;
  bool ok;
  switch (a.d / 16) {
    case 1: ok = launch_decode<1>(a, groups, stream); break;
    case 2: ok = launch_decode<2>(a, groups, stream); break;
    case 3: ok = launch_decode<3>(a, groups, stream); break;
    case 4: ok = launch_decode<4>(a, groups, stream); break;
    case 5: ok = launch_decode<5>(a, groups, stream); break;
    case 6: ok = launch_decode<6>(a, groups, stream); break;
    case 7: ok = launch_decode<7>(a, groups, stream); break;
    default: ok = launch_decode<8>(a, groups, stream); break;
  }
  TK_REQUIRE(ok, "decode_layers: the kernel's local memory could not be reserved");
  TK_CHECK_LAUNCH("decode_layers");
  return 0;
}
