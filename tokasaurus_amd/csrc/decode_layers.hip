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
// through the caches (agent-scope relaxed atomics), because each of the chip's eight dies has
// an L2 of its own; the grid barrier then needs no cache-wide write-back, only a wait for the
// workgroup's own stores.  It is read with ordinary cached loads, which is sound because every
// block has scratch buffers of its own: within a launch a buffer is written once and read only
// behind the barrier that follows, so no cache can hold a line of it from before the write (and
// a launch starts with clean caches).  Reading around the caches instead would send every
// workgroup's read of the same few KB to the one or two memory channels that hold them.
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
#include "attention_merge.h"

#define DL_WAVES 8            // wavefronts of a workgroup
#define DL_THREADS (64 * DL_WAVES)
#define DL_RING 8             // (tile, step) slots whose loads a wavefront keeps in flight
#define DL_MAX_TILES 4        // 16-row tiles (or tile pairs) a workgroup may own in one phase
#define DL_FAN 16             // workgroups per first-level counter of the barrier
#define DL_MAX_GROUPS 4096    // workgroups a launch may have
#define DL_MAX_TABLES 4       // block tables (cache groups) a run of blocks may use
#define DL_MARKS_PER_LAYER 24  // timing marks a block may leave

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
  // scratch, one buffer a block each (a buffer is written once in a launch):
  bf16_t* xs;   // [n_layers + 1][M, H] the residual stream: xs[0] in, xs[l + 1] out of block l
  bf16_t* xbs;  // [n_layers][M, H] the stream between mixer and feed-forward
  bf16_t* qs;   // [n_layers][M, nq d]
  bf16_t* hs;   // [n_layers][M, I]
  float* part_o;   // [n_layers][M][nkv][max_splits][16][d] partial attention results
  float* part_ml;  // [n_layers][M][nkv][max_splits][16][2]
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
  // diagnostics (null: none): workgroup `timing_group` writes pairs (mark id, constant-rate clock
  // of 100 MHz) at the start and at up to DL_MARKS_PER_LAYER places of every block:
  // 2 * (1 + DL_MARKS_PER_LAYER * n_layers) words
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
// (the output product keeps the merged attention, its operand, behind the sums)
#define DL_SSQ_FLOATS (DL_WAVES * 16)
#define DL_RED_FLOATS (DL_MAX_TILES * DL_WAVES * 64 * 4)

struct PhaseShape {
  int u0, u1, nt, th;  // this workgroup's units [u0, u1), in nt tiles of th units
};

// Diagnostics: one thread of one workgroup leaves (id, clock) pairs.
struct Marks {
  unsigned long long* out;  // null: off
  int at, limit;
  __device__ __forceinline__ void operator()(int id) {
    if (out != nullptr && at < limit) {
      out[2 * at] = (unsigned long long)id;
      out[2 * at + 1] = wall_clock64();
      ++at;
    }
  }
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

// One wavefront's share of a product phase.  C[token][unit] = sum_k A[token][k] W[row(unit)][k]
// for the workgroup's units; the wavefront takes the steps ks0 .. ks0 + n_steps - 1 of K (32
// values a step) of every tile: n_slots = nt * n_steps (tile, step) slots, in chunks of 8.
//   PAIRED: a unit is two rows, row(unit) and row(unit) + pair_off; `half` > 0 maps unit u to
//   row (u / half) * 2 half + u % half (the first of a rotation's pair), else row = unit.
#define DL_CHUNK 8
struct Share {
  const bf16_t* W;
  const bf16_t* zeros;  // 16 bytes of zeros in device memory: what a lane without a weight row reads
  PhaseShape p;
  int K, half, pair_off, ks0, n_steps, n_slots, n_chunks;
};

__device__ __forceinline__ Share make_share(const bf16_t* W, const bf16_t* zeros, int K, int units, int half, int pair_off,
                                            int wave) {
  Share s;
  s.W = W; s.zeros = zeros; s.K = K; s.half = half; s.pair_off = pair_off;
  s.p = phase_shape(units);
  const int K32 = (K + 31) >> 5;
  s.ks0 = K32 * wave / DL_WAVES;
  s.n_steps = K32 * (wave + 1) / DL_WAVES - s.ks0;
  s.n_slots = s.p.nt * s.n_steps;
  s.n_chunks = (s.n_slots + DL_CHUNK - 1) / DL_CHUNK;
  return s;
}

template <bool PAIRED>
struct WChunk {
  bf16x8_t a[DL_CHUNK];
  bf16x8_t b[PAIRED ? DL_CHUNK : 1];
};

__device__ __forceinline__ bf16x8_t keep_if(bool ok, bf16x8_t v) {
  union { bf16x8_t v; uint32_t u[4]; } x;
  x.v = v;
#pragma unroll
  for (int e = 0; e < 4; ++e) x.u[e] = ok ? x.u[e] : 0u;
  return x.v;
}

// The weights of chunk `chunk`: every lane loads, from an address that always exists (a slot or
// a lane without a weight row reads 16 bytes of zeros), so that the loads of a chunk are
// straight-line code whose arrival the hardware's counter tells apart, and nothing has to
// touch a loaded value before the matrix core does.
template <bool PAIRED>
__device__ __forceinline__ void load_weights(WChunk<PAIRED>& c, const Share& s, int chunk, int r, int q) {
  const int n_steps = max(s.n_steps, 1);
  int tile = chunk * DL_CHUNK / n_steps, si = chunk * DL_CHUNK - tile * n_steps;
#pragma unroll
  for (int j = 0; j < DL_CHUNK; ++j) {
    const int unit = s.p.u0 + tile * s.p.th + r, k0 = (s.ks0 + si) * 32 + q * 8;
    const bool ok = tile < s.p.nt && r < s.p.th && unit < s.p.u1 && k0 < s.K;
    const int uu = ok ? unit : 0;
    const int row = s.half > 0 ? (uu / s.half) * (2 * s.half) + uu % s.half : uu;
    const bf16_t* ptr = s.W + (size_t)row * s.K + k0;
    c.a[j] = *(const bf16x8_t*)(ok ? ptr : s.zeros);
    if (PAIRED) c.b[j] = *(const bf16x8_t*)(ok ? ptr + (size_t)s.pair_off * s.K : s.zeros);
    if (++si == n_steps) { si = 0; ++tile; }
  }
}

template <bool PAIRED>
__device__ __forceinline__ void zero_weights(WChunk<PAIRED>& c) {
#pragma unroll
  for (int j = 0; j < DL_CHUNK; ++j) {
    c.a[j] = dl_zero8();
    if (PAIRED) c.b[j] = dl_zero8();
  }
}

// The weights of a share, NB chunks deep.  begin() asks for the first NB chunks and may be called
// long before the product runs (before the barrier that the product's other operand waits for:
// weights do not depend on it); the product asks for chunk c + NB when it has multiplied chunk c.
template <bool PAIRED, int NB>
struct WeightStream {
  WChunk<PAIRED> buf[NB];
  Share s;
  __device__ __forceinline__ void begin(const bf16_t* W, const bf16_t* zeros, int K, int units, int half, int pair_off,
                                        int wave, int r, int q) {
    s = make_share(W, zeros, K, units, half, pair_off, wave);
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      if (i < s.n_chunks) load_weights<PAIRED>(buf[i], s, i, r, q);
      else zero_weights<PAIRED>(buf[i]);
    }
  }
};

// The product of a stream whose first chunks begin() has asked for.
//   load_a(step, first_pass) gives lane (token r, quarter q) its 8 values A[r][32 step + 8 q ..]
//   for ANY step (it reads an address that exists and drops what lies past the end);
//   first_pass is true in the workgroup's first tile (statistics of A are taken there, once).
//   The operands of a chunk are asked for while the chunk before it is multiplied.
//   before_sync(): called by every wavefront after its last product, before the workgroup's
//   barrier (statistics go to LDS here; the next phase's weights are asked for here).
//   epilogue(token, slot, unit0, limit, s0, s1): the sums of units unit0 .. unit0 + 3 (those
//   below `limit` exist) for one token, s1 the paired rows'; slot = tile * 4 + quarter numbers
//   the calls of one token.
template <bool PAIRED, int NB, typename LoadA, typename BeforeSync, typename Epilogue>
__device__ __forceinline__ void product_run(WeightStream<PAIRED, NB>& ws, float* lds, Marks& mark, int mark_id, int r, int q,
                                            LoadA load_a, BeforeSync before_sync, Epilogue epilogue) {
  static_assert(NB == 1 || NB % 2 == 0, "the operand buffers alternate: an even number of weight buffers, or one");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Share s = ws.s;
  const PhaseShape p = s.p;
  const int n_steps = max(s.n_steps, 1);
  f32x4_t* red = (f32x4_t*)(lds + DL_SSQ_FLOATS);
  f32x4_t* red2 = red + p.nt * DL_WAVES * 64;

  bf16x8_t av[2][DL_CHUNK];
  auto load_operands = [&](bf16x8_t (&dst)[DL_CHUNK], int chunk) {
    int tile = chunk * DL_CHUNK / n_steps, si = chunk * DL_CHUNK - tile * n_steps;
#pragma unroll
    for (int j = 0; j < DL_CHUNK; ++j) {
      dst[j] = load_a(s.ks0 + si, tile == 0);
      if (++si == n_steps) { si = 0; ++tile; }
    }
  };
  f32x4_t acc0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, acc1 = acc0;
  int c_tile = 0, c_step = 0;
  auto multiply = [&](const WChunk<PAIRED>& w, const bf16x8_t (&a)[DL_CHUNK], int chunk) {
#pragma unroll
    for (int j = 0; j < DL_CHUNK; ++j) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.a[j], a[j], acc0, 0, 0, 0);
      if (PAIRED) acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.b[PAIRED ? j : 0], a[j], acc1, 0, 0, 0);
      if (chunk * DL_CHUNK + j < s.n_slots && ++c_step == s.n_steps) {
        red[(c_tile * DL_WAVES + wave) * 64 + lane] = acc0;
        if (PAIRED) red2[(c_tile * DL_WAVES + wave) * 64 + lane] = acc1;
        acc0 = f32x4_t{0.f, 0.f, 0.f, 0.f};
        acc1 = acc0;
        c_step = 0;
        ++c_tile;
      }
    }
  };

  if (s.n_chunks > 0) load_operands(av[0], 0);
  for (int c = 0; c < s.n_chunks; c += (NB == 1 ? 2 : NB)) {
#pragma unroll
    for (int i = 0; i < (NB == 1 ? 2 : NB); ++i) {
      if (c + i < s.n_chunks) {
        if (c + i + 1 < s.n_chunks) load_operands(av[(i + 1) & 1], c + i + 1);
        multiply(ws.buf[i % NB], av[i & 1], c + i);
        if (c + i + NB < s.n_chunks) load_weights<PAIRED>(ws.buf[i % NB], s, c + i + NB, r, q);
      }
    }
  }
  if (s.n_steps == 0) {
    // a wavefront without a part of K still owes its (zero) sums
    for (int t = 0; t < p.nt; ++t) {
      red[(t * DL_WAVES + wave) * 64 + lane] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (PAIRED) red2[(t * DL_WAVES + wave) * 64 + lane] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  }
  mark(mark_id);  // products done
  before_sync();
  __syncthreads();
  mark(mark_id + 1);  // sums of all wavefronts in LDS
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
__device__ __forceinline__ bf16x8_t load_rows(const bf16_t* A, const bf16_t* zeros, int lda, int M, int K, int step, int r,
                                              int q) {
  const int k0 = step * 32 + q * 8;
  const bool ok = r < M && k0 < K;
  return *(const bf16x8_t*)(ok ? A + (size_t)r * lda + k0 : zeros);
}

// The operand of a product behind an RMSNorm: x * w rounded once (the rows are divided by their
// rms after the product), and the sum of x^2 over what this lane saw.
__device__ __forceinline__ bf16x8_t load_normed(const bf16_t* x, const bf16_t* zeros, int H, int M, const void* w, int w_f32,
                                                int step, int r, int q, bool first, float& ssq) {
  const int k0 = step * 32 + q * 8;
  const bool ok = r < M && k0 < H;
  const int kk = ok ? k0 : 0;
  union { uint4 u; uint16_t h[8]; } xv;
  const bf16_t* xp = ok ? x + (size_t)r * H + k0 : zeros;
  xv.u = *(const uint4*)xp;
  float wv[8];
  if (w_f32) {
    const f32x4_t a = *(const f32x4_t*)((const float*)w + kk), b = *(const f32x4_t*)((const float*)w + kk + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { wv[e] = a[e]; wv[4 + e] = b[e]; }
  } else {
    union { uint4 u; uint16_t h[8]; } ww;
    ww.u = *(const uint4*)((const bf16_t*)w + kk);
#pragma unroll
    for (int e = 0; e < 8; ++e) wv[e] = bf16_bits_to_f32(ww.h[e]);
  }
  bf16x8_t out;
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float xr = bf16_bits_to_f32(xv.h[e]);
    ss = fmaf(xr, xr, ss);
    out[e] = (__bf16)(wv[e] * xr);
  }
  if (first) ssq += ss;
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

// four values of a bfloat16 row that other workgroups wrote (those below `limit`; else 0)
__device__ __forceinline__ void load_row4(const bf16_t* row, int n, int limit, float (&o)[4]) {
  if (n + 3 < limit && (n & 3) == 0 && (((uintptr_t)row) & 7) == 0) {
    union { uint64_t u; uint16_t h[4]; } pk;
    pk.u = *(const uint64_t*)(row + n);
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = bf16_bits_to_f32(pk.h[j]);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[j] = 0.f;
      if (n + j < limit) o[j] = __bfloat162float(row[n + j]);
    }
  }
}

// A value the compiler must take as new: what is computed from it inside the loop over the
// blocks stays inside that loop.  Without this the addresses and masks of every phase, which
// do not change from block to block, are all computed ahead of the loop and kept, in far more
// registers than a wavefront has; they come back from scratch memory in the middle of the
// products, where every such load waits for all the weights asked for before it.
__device__ __forceinline__ int per_block(int x) {
  asm volatile("" : "+s"(x));
  return x;
}

// ---------------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------------
// chunks (of 8 slots) of weights a wavefront asks for ahead, per product
#define DL_AHEAD_QKV 1
#define DL_AHEAD_O 1
#define DL_AHEAD_GU 1
#define DL_AHEAD_DOWN 2

template <int DT, bool BIG>
__global__ __launch_bounds__(DL_THREADS) void decode_layers_kernel(DecodeArgs a) {
  extern __shared__ __align__(16) float lds[];
  constexpr int D = DT * 16;
  const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, q = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int half = D / 2;
  GridSync gs = grid_sync_begin(a);
  const bf16_t* zeros = (const bf16_t*)(a.sync + 4);  // words 4 .. 7 of the sync buffer are never written
  Marks mark;
  mark.out = (a.timing != nullptr && (int)blockIdx.x == a.timing_group && tid == 0) ? a.timing : nullptr;
  mark.at = 0;
  mark.limit = 1 + DL_MARKS_PER_LAYER * a.n_layers;
  mark(0);

  WeightStream<true, DL_AHEAD_QKV> w_qkv;
  WeightStream<false, DL_AHEAD_O> w_o;
  WeightStream<true, DL_AHEAD_GU> w_gu;
  WeightStream<false, DL_AHEAD_DOWN> w_down;

  for (int li = 0; li < a.n_layers; ++li) {
    const int M = per_block(a.M), H = per_block(a.H), I = per_block(a.I), nq = per_block(a.nq), nkv = per_block(a.nkv),
              P = per_block(a.P);
    const int group = nq / nkv;
    const DecodeLayer L = a.layers[li];
    const int* table = a.tables[L.table];
    const int table_stride = a.table_stride[L.table];
    const bool last_layer = li + 1 == a.n_layers;
    // this block's scratch
    const bf16_t* x_in = a.xs + (size_t)li * M * H;
    bf16_t* x_out = a.xs + (size_t)(li + 1) * M * H;
    bf16_t* xb = a.xbs + (size_t)li * M * H;
    bf16_t* qbuf = a.qs + (size_t)li * M * nq * D;
    bf16_t* hbuf = a.hs + (size_t)li * M * I;
    const size_t part_items = (size_t)M * nkv * a.max_splits * 16;
    float* part_o = a.part_o + (size_t)li * part_items * D;
    float* part_ml = a.part_ml + (size_t)li * part_items * 2;

    // ---- 1. q | k | v of the normed stream, rotated; q to scratch, k and v to the pages
    {
      w_qkv.begin(L.w_qkv, zeros, H, (nq + 2 * nkv) * half, half, half, wave, r, q);
      // what the rotation of this thread's first four units reads, asked for ahead of the product
      const PhaseShape shape = w_qkv.s.p;
      int pre_pos = 0, pre_page = 0;
      float pre_cs[4] = {1.f, 1.f, 1.f, 1.f}, pre_sn[4] = {0.f, 0.f, 0.f, 0.f};
      if (tid < shape.nt * 64 && (tid & 15) < M) {
        const int token = tid & 15;
        pre_pos = a.positions[token];
        pre_page = table[(size_t)token * table_stride + pre_pos / P];
        const int unit0 = shape.u0 + (tid >> 6) * shape.th + ((tid & 63) >> 4) * 4;
        const int limit = min(shape.u1, shape.u0 + ((tid >> 6) + 1) * shape.th);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int unit = unit0 + j;
          if (unit < limit && unit / half < nq + nkv && L.cos_t != nullptr) {
            pre_cs[j] = L.cos_t[(size_t)pre_pos * half + unit % half];
            pre_sn[j] = L.sin_t[(size_t)pre_pos * half + unit % half];
          }
        }
      }
      float ssq = 0.f;
      product_run(
          w_qkv, lds, mark, 10, r, q,
          [&](int step, bool first) { return load_normed(x_in, zeros, H, M, L.norm1, L.norm1_f32, step, r, q, first, ssq); },
          [&]() { put_ssq(lds, ssq, wave, lane); },
          [&](int token, int slot, int unit0, int limit, f32x4_t s0, f32x4_t s1) {
            if (token >= M) return;
            const float rstd = rstd_of(lds, token, H, L.eps1);
            // this thread's first call is the one it asked ahead for: (tile, quarter, token) = its own thread number
            const bool pre = (slot >> 2) * 64 + (slot & 3) * 16 + token == tid;
            const int pos = pre ? pre_pos : a.positions[token];
            const int page = pre ? pre_page : table[(size_t)token * table_stride + pos / P];
            const int off = pos % P;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int unit = unit0 + j;
              if (unit >= limit) continue;
              const int head = unit / half, c = unit - head * half;
              const float x1 = round_to<bf16_t>(s0[j] * rstd), x2 = round_to<bf16_t>(s1[j] * rstd);
              float o1 = x1, o2 = x2;
              if (head < nq + nkv && L.cos_t != nullptr) {
                const float cs = pre ? pre_cs[j] : L.cos_t[(size_t)pos * half + c];
                const float sn = pre ? pre_sn[j] : L.sin_t[(size_t)pos * half + c];
                rotate_pair(x1, x2, cs, sn, o1, o2);
              }
              if (head < nq) {
                bf16_t* dst = qbuf + (size_t)token * (nq * D) + (size_t)head * D + c;
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
    mark(12);
    grid_barrier(gs, false);
    mark(13);

    // ---- 2. attention of every (request, kv head) over its pages, the keys cut into splits
    {
      AttnArgs at;
      at.q = qbuf; at.q_stride = nq * D; at.out = nullptr; at.out_stride = 0;
      at.kcache = L.kcache; at.vcache = L.vcache;
      at.block_table = table; at.table_stride = table_stride;
      at.q_start = nullptr; at.kv_len = a.kv_len; at.tile_req = nullptr; at.tile_row0 = nullptr; at.tile_row1 = nullptr;
      at.n_tiles = M; at.nq = nq; at.nkv = nkv; at.group = group; at.P = P; at.window = L.window;
      at.p_shift = 31 - __builtin_clz(P);
      at.scale_log2 = a.scale * 1.4426950408889634f;
      at.split = a.split; at.max_splits = a.max_splits; at.part_o = part_o; at.part_ml = part_ml;
      const int n_items = M * nkv * a.max_splits;
      for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int split_index = item % a.max_splits, rest = item / a.max_splits;
        attention_item<DT, 1, BIG, true>(at, rest / nkv, rest % nkv, split_index, lds, DL_WAVES);
        __syncthreads();  // the next item uses the same LDS
      }
      mark(21);
    }
    mark(22);
    grid_barrier(gs, false);
    mark(23);

    // ---- 3. xb = x + attention * Wo^T; the attention's splits are merged on the way in
    {
      bf16_t* stage = (bf16_t*)(lds + DL_SSQ_FLOATS + DL_RED_FLOATS);
      w_o.begin(L.w_o, zeros, nq * D, H, 0, 0, wave, r, q);
      MergeArgs mg;
      mg.part_o = part_o; mg.part_ml = part_ml; mg.kv_len = a.kv_len;
      mg.M = M; mg.nq = nq; mg.nkv = nkv; mg.D = D; mg.split = a.split; mg.max_splits = a.max_splits; mg.window = L.window;
      merge_attention_to_lds(mg, stage, DL_THREADS);
      __syncthreads();
      mark(29);
      product_run(
          w_o, lds, mark, 30, r, q,
          [&](int step, bool) { return *(const bf16x8_t*)(stage + (size_t)(min(step, (nq * D + 31) / 32 - 1) * 64 + lane) * 8); },
          [&]() {},
          [&](int token, int, int unit0, int limit, f32x4_t s0, f32x4_t) {
            if (token >= M) return;
            float o[4], res[4];
            load_row4(x_in + (size_t)token * H, unit0, limit, res);
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = round_to<bf16_t>(s0[j]) + res[j];
            store_row4(xb + (size_t)token * H, unit0, limit, o);
          });
    }
    mark(32);
    grid_barrier(gs, false);
    mark(33);

    // ---- 4. h = silu(gate) * up of the normed stream
    {
      w_gu.begin(L.w_gu, zeros, H, I, 0, I, wave, r, q);
      float ssq = 0.f;
      product_run(
          w_gu, lds, mark, 40, r, q,
          [&](int step, bool first) { return load_normed(xb, zeros, H, M, L.norm2, L.norm2_f32, step, r, q, first, ssq); },
          [&]() { put_ssq(lds, ssq, wave, lane); },
          [&](int token, int, int unit0, int limit, f32x4_t s0, f32x4_t s1) {
            if (token >= M) return;
            const float rstd = rstd_of(lds, token, H, L.eps2);
            float o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = silu_mul_bf16(s0[j] * rstd, s1[j] * rstd);
            store_row4(hbuf + (size_t)token * I, unit0, limit, o);
          });
    }
    mark(42);
    grid_barrier(gs, false);
    mark(43);

    // ---- 5. x = xb + h * Wdown^T (and, after the last block, what the following norm needs)
    {
      float* emit_part = lds + DL_SSQ_FLOATS + DL_RED_FLOATS;  // [tile * 4 + quarter][16 tokens], behind the sums
      const bool emit = last_layer && a.emit_w != nullptr;
      w_down.begin(L.w_down, zeros, I, H, 0, 0, wave, r, q);
      const PhaseShape shape = w_down.s.p;
      product_run(
          w_down, lds, mark, 50, r, q,
          [&](int step, bool) { return load_rows(hbuf, zeros, I, M, I, step, r, q); },
          [&]() {},
          [&](int token, int slot, int unit0, int limit, f32x4_t s0, f32x4_t) {
            float o[4] = {0.f, 0.f, 0.f, 0.f}, ss = 0.f;
            if (token < M) {
              float res[4];
              load_row4(xb + (size_t)token * H, unit0, limit, res);
#pragma unroll
              for (int j = 0; j < 4; ++j) o[j] = round_to<bf16_t>(s0[j]) + res[j];
              store_row4(x_out + (size_t)token * H, unit0, limit, o);
            }
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
    mark(52);
    grid_barrier(gs, last_layer);
    mark(53);
  }
}

// ---------------------------------------------------------------------------------
// launch
// ---------------------------------------------------------------------------------
static size_t decode_lds_bytes(int d, int nq) {
  const size_t product = sizeof(float) * (DL_SSQ_FLOATS + (size_t)2 * DL_RED_FLOATS);
  const size_t emit = sizeof(float) * (DL_SSQ_FLOATS + (size_t)DL_RED_FLOATS + DL_MAX_TILES * 4 * 16);
  // the output product: its sums, and behind them the merged attention, 1 KB a step of 32
  const size_t merged = sizeof(float) * (DL_SSQ_FLOATS + (size_t)DL_RED_FLOATS) + (size_t)((nq * d + 31) / 32) * 1024;
  const size_t attention = sizeof(float) * (size_t)DL_WAVES * 16 * (d + 4);
  size_t n = product > emit ? product : emit;
  n = n > merged ? n : merged;
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
  const size_t lds = decode_lds_bytes(DT * 16, a.nq);
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
  TK_REQUIRE(d == 16 || d == 32 || d == 64 || d == 128, "decode_layers: head size %d is not 16, 32, 64 or 128", d);
  TK_REQUIRE(P >= 4 && (P & (P - 1)) == 0, "decode_layers: page size %d is not a power of two from 4", P);
  TK_REQUIRE(H > 0 && I > 0 && H % 8 == 0 && I % 8 == 0, "decode_layers: widths %d and %d must be multiples of 8", H, I);
  TK_REQUIRE(groups >= 1 && groups <= DL_MAX_GROUPS, "decode_layers: %d workgroups", groups);
  const int limit = 16 * DL_MAX_TILES;
  const int units[4] = {(nq + 2 * nkv) * (d / 2), H, I, H};
  for (int i = 0; i < 4; ++i)
    TK_REQUIRE((units[i] + groups - 1) / groups <= limit,
               "decode_layers: %d outputs over %d workgroups are more than %d each", units[i], groups, limit);
  TK_REQUIRE(decode_lds_bytes(d, nq) <= 160 * 1024, "decode_layers: %d heads of size %d do not fit the local memory", nq, d);
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
  TK_REQUIRE(a.positions && a.kv_len && a.xs && a.xbs && a.qs && a.hs && a.part_o && a.part_ml && a.sync && a.status,
             "decode_layers: an operand is missing");
  TK_REQUIRE(a.split > 0 && a.split % (32 * DL_WAVES) == 0 && a.max_splits >= 1,
             "decode_layers: a split of %d keys is no multiple of %d", a.split, 32 * DL_WAVES);
  TK_REQUIRE(a.scale > 0.f, "decode_layers: the scale must be positive");
  TK_REQUIRE((((uintptr_t)a.xs | (uintptr_t)a.xbs | (uintptr_t)a.qs | (uintptr_t)a.hs | (uintptr_t)a.part_o |
               (uintptr_t)a.part_ml) & 15) == 0, "decode_layers: operands must be 16-byte aligned");
  TK_REQUIRE(a.emit_w == nullptr || (a.emit_scaled && a.emit_sumsq), "decode_layers: outputs for the following norm are missing");
  TK_REQUIRE(a.spin_cap > 0, "decode_layers: the spin limit must be positive");
  if (a.expect_groups == 0) a.expect_groups = (uint32_t)groups;
  if (a.n_layers == 0) return 0;
  // built for the head sizes 16, 32, 64 and 128 (each instance is a large kernel); others are
  // refused by tk_decode_layers_supports and run through the separate kernels
  bool ok;
  switch (a.d / 16) {
    case 1: ok = launch_decode<1>(a, groups, stream); break;
    case 2: ok = launch_decode<2>(a, groups, stream); break;
    case 4: ok = launch_decode<4>(a, groups, stream); break;
    case 8: ok = launch_decode<8>(a, groups, stream); break;
    default: TK_REQUIRE(false, "decode_layers: no kernel was built for head size %d", a.d);
  }
  TK_REQUIRE(ok, "decode_layers: the kernel's local memory could not be reserved");
  TK_CHECK_LAUNCH("decode_layers");
  return 0;
}
