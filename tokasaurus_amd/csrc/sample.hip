// Sampling from 32-bit logits:
//   temperature == 0: the index of the largest raw logit (the lowest index on a tie);
//   temperature  > 0: p = softmax(logits / T) and the smallest index whose
//                     cumulative probability exceeds the row's uniform number u.
// Also the chosen token's log-probability under p (T treated as 1 when 0), and
// optionally the token written to the request's slot for the next step's embedding.
//
// Two kernels, so that a few rows of a large vocabulary still fill the chip:
//   sample_partial: one workgroup per (row, chunk of SM_CHUNK logits): the chunk's
//                   maximum, its first index, and sum exp((x - max) / T);
//   sample_finish:  one workgroup per row: joins the chunks in chunk order, finds
//                   the chunk in which the cumulative mass passes u, and scans it.
#include "common.h"
#include "sample.h"

#include <mutex>

#define SM_THREADS 256
#define SM_PER_THREAD 8
#define SM_CHUNK (SM_THREADS * SM_PER_THREAD)
#define SM_MAX_CHUNKS 4096

__global__ __launch_bounds__(SM_THREADS) void sample_partial_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
    float* __restrict__ part_max, float* __restrict__ part_sum, int* __restrict__ part_arg,
    int n_chunks) {
  __shared__ float red[16];
  __shared__ int red_i[16];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & (TK_WAVE - 1), wave = tid / TK_WAVE;
  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row];
  const float inv_t = T > 0.f ? 1.0f / T : 1.0f;
  const int begin = chunk * SM_CHUNK + tid * SM_PER_THREAD;
  float v[SM_PER_THREAD];
  float best = -INFINITY;
  int best_i = vocab;
#pragma unroll
  for (int i = 0; i < SM_PER_THREAD; ++i) {
    v[i] = begin + i < vocab ? x[begin + i] : -INFINITY;
    if (v[i] > best) { best = v[i]; best_i = begin + i; }
  }
  float m = best;
  int mi = best_i;
#pragma unroll
  for (int o = TK_WAVE / 2; o > 0; o >>= 1) {
    const float om = __shfl_xor(m, o, TK_WAVE);
    const int oi = __shfl_xor(mi, o, TK_WAVE);
    if (om > m || (om == m && oi < mi)) { m = om; mi = oi; }
  }
  if (lane == 0) { red[wave] = m; red_i[wave] = mi; }
  __syncthreads();
  m = red[0]; mi = red_i[0];
  for (int w = 1; w < SM_THREADS / TK_WAVE; ++w)
    if (red[w] > m || (red[w] == m && red_i[w] < mi)) { m = red[w]; mi = red_i[w]; }
  float local = 0.f;
#pragma unroll
  for (int i = 0; i < SM_PER_THREAD; ++i) local += (v[i] == -INFINITY) ? 0.f : expf((v[i] - m) * inv_t);
  const float total = block_sum(local, red);
  if (tid == 0) {
    const size_t o = (size_t)row * n_chunks + chunk;
    part_max[o] = m;
    part_sum[o] = total;
    part_arg[o] = mi;
  }
}

__global__ __launch_bounds__(SM_THREADS) void sample_finish_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
    const float* __restrict__ uniform, const float* __restrict__ part_max,
    const float* __restrict__ part_sum, const int* __restrict__ part_arg, int n_chunks,
    const int* __restrict__ slots, int* __restrict__ last_token, int* __restrict__ out_ids,
    float* __restrict__ out_logprobs) {
  __shared__ float cum[SM_MAX_CHUNKS];  // mass of chunks 0..c relative to the row maximum
  __shared__ float red[16];
  __shared__ float wave_tot[16];
  __shared__ float row_max_s, total_s;
  __shared__ int argmax_s, pick_chunk, chosen;
  const int row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & (TK_WAVE - 1), wave = tid / TK_WAVE;
  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row];
  const float inv_t = T > 0.f ? 1.0f / T : 1.0f;
  const float* pm = part_max + (size_t)row * n_chunks;
  const float* ps = part_sum + (size_t)row * n_chunks;
  const int* pa = part_arg + (size_t)row * n_chunks;

  // the row's maximum and its first index
  float m = -INFINITY;
  int mi = vocab;
  for (int c = tid; c < n_chunks; c += SM_THREADS) {
    const float cm = pm[c];
    const int ci = pa[c];
    if (cm > m || (cm == m && ci < mi)) { m = cm; mi = ci; }
  }
#pragma unroll
  for (int o = TK_WAVE / 2; o > 0; o >>= 1) {
    const float om = __shfl_xor(m, o, TK_WAVE);
    const int oi = __shfl_xor(mi, o, TK_WAVE);
    if (om > m || (om == m && oi < mi)) { m = om; mi = oi; }
  }
  __shared__ int red_i[16];
  if (lane == 0) { red[wave] = m; red_i[wave] = mi; }
  __syncthreads();
  if (tid == 0) {
    float bm = red[0];
    int bi = red_i[0];
    for (int w = 1; w < SM_THREADS / TK_WAVE; ++w)
      if (red[w] > bm || (red[w] == bm && red_i[w] < bi)) { bm = red[w]; bi = red_i[w]; }
    row_max_s = bm;
    argmax_s = bi;
  }
  __syncthreads();
  const float row_max = row_max_s;
  // every chunk's mass relative to the row maximum, then the running sum in chunk order
  for (int c = tid; c < n_chunks; c += SM_THREADS) cum[c] = ps[c] * expf((pm[c] - row_max) * inv_t);
  __syncthreads();
  if (tid == 0) {
    float run = 0.f;
    for (int c = 0; c < n_chunks; ++c) { run += cum[c]; cum[c] = run; }
    total_s = run;
    pick_chunk = n_chunks - 1;
    chosen = (T > 0.f) ? vocab - 1 : argmax_s;
  }
  __syncthreads();
  const float total = total_s;
  if (T > 0.f) {
    const float target = uniform[row] * total;
    for (int c = tid; c < n_chunks; c += SM_THREADS) {
      const float lower = c > 0 ? cum[c - 1] : 0.f;
      if (lower <= target && target < cum[c]) atomicMin(&pick_chunk, c);
    }
    __syncthreads();
    const int c = pick_chunk;
    const float base = c > 0 ? cum[c - 1] : 0.f;
    const int begin = c * SM_CHUNK + tid * SM_PER_THREAD;
    float e[SM_PER_THREAD];
    float local = 0.f;
#pragma unroll
    for (int i = 0; i < SM_PER_THREAD; ++i) {
      e[i] = begin + i < vocab ? expf((x[begin + i] - row_max) * inv_t) : 0.f;
      local += e[i];
    }
    float scan = local;  // inclusive scan over the threads, in thread order
#pragma unroll
    for (int o = 1; o < TK_WAVE; o <<= 1) {
      const float up = __shfl_up(scan, o, TK_WAVE);
      if (lane >= o) scan += up;
    }
    if (lane == TK_WAVE - 1) wave_tot[wave] = scan;
    __syncthreads();
    float before = base;
    for (int w = 0; w < wave; ++w) before += wave_tot[w];
    const float upper = before + scan, lower = upper - local;
    // the last element of the chunk takes what rounding leaves over
    const bool last_thread = begin < vocab && begin + SM_PER_THREAD >= min(vocab, (c + 1) * SM_CHUNK);
    if (begin < vocab && lower <= target && (target < upper || last_thread)) {
      float run = lower;
      int pick = min(begin + SM_PER_THREAD, vocab) - 1;
#pragma unroll
      for (int i = 0; i < SM_PER_THREAD; ++i) {
        run += e[i];
        if (run > target && begin + i < vocab) { pick = min(pick, begin + i); }
      }
      atomicMin(&chosen, pick);
    }
    __syncthreads();
  }
  if (tid == 0) {
    const int id = chosen;
    out_ids[row] = id;
    if (out_logprobs) out_logprobs[row] = (x[id] - row_max) * inv_t - logf(total);
    if (last_token && slots) last_token[slots[row]] = id;
  }
}

TK_API int tk_sample_chunks(int vocab) { return (vocab + SM_CHUNK - 1) / SM_CHUNK; }

// The two launches of the sampler on checked arguments.
static int launch_sample(const float* logits, int ld, int rows, int vocab, const float* temperature,
                         const float* uniform, const int* slots, int* last_token, int* out_ids,
                         float* out_logprobs, float* part_max, float* part_sum, int* part_arg,
                         int n_chunks, hipStream_t stream) {
  hipLaunchKernelGGL(sample_partial_kernel, dim3(n_chunks, rows), dim3(SM_THREADS), 0, stream, logits,
                     ld, vocab, temperature, part_max, part_sum, part_arg, n_chunks);
  TK_CHECK_LAUNCH("sample_partial");
  hipLaunchKernelGGL(sample_finish_kernel, dim3(rows), dim3(SM_THREADS), 0, stream, logits, ld, vocab,
                     temperature, uniform, part_max, part_sum, part_arg, n_chunks, slots, last_token,
                     out_ids, out_logprobs);
  TK_CHECK_LAUNCH("sample_finish");
  return 0;
}

// part_max, part_sum (float) and part_arg (int) hold rows * tk_sample_chunks(vocab) entries each.
TK_API int tk_sample(const float* logits, int ld, int rows, int vocab, const float* temperature,
                         const float* uniform, const int* slots, int* last_token, int* out_ids,
                         float* out_logprobs, float* part_max, float* part_sum, int* part_arg,
                         hipStream_t stream) {
  TK_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d vocab=%d ld=%d", rows,
             vocab, ld);
  const int n_chunks = (vocab + SM_CHUNK - 1) / SM_CHUNK;
  TK_REQUIRE(n_chunks <= SM_MAX_CHUNKS, "sample: a vocabulary of %d is larger than %d", vocab,
             SM_MAX_CHUNKS * SM_CHUNK);
  TK_REQUIRE(rows < 65536, "sample: %d rows are too many for one call", rows);
  TK_REQUIRE(part_max && part_sum && part_arg, "sample: scratch missing");
  if (rows == 0) return 0;
  return launch_sample(logits, ld, rows, vocab, temperature, uniform, slots, last_token, out_ids, out_logprobs,
                       part_max, part_sum, part_arg, n_chunks, stream);
}

// ---------------------------------------------------------------------------
// tk_sample_static: the partial results in a device array of the library's own (sample.h).
// In host code the array's name is only a handle: its address on a GPU comes from
// hipGetSymbolAddress, asked once per device with that device current (every GPU has a copy
// of the array at an address of its own), and only that address is given to kernels.
#define SAMPLE_STATIC_DEVICES 64
static __device__ __align__(256) uint32_t scratch[3 * TK_SAMPLE_STATIC_ITEMS];
static void* g_scratch_ptr[SAMPLE_STATIC_DEVICES];
static std::mutex g_scratch_mutex;

// The array's address on the current device (null, with the error text set, on failure).
static uint32_t* static_scratch() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= SAMPLE_STATIC_DEVICES) {
    tk_set_error("sample_static: no usable current device (%s, device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      tk_set_error("sample_static: the scratch array has no address on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return (uint32_t*)g_scratch_ptr[dev];
}

TK_API int tk_sample_static(const float* logits, int ld, int rows, int vocab, const float* temperature,
                            const float* uniform, const int* slots, int* last_token, int* out_ids,
                            float* out_logprobs, hipStream_t stream) {
  TK_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample_static: bad sizes rows=%d vocab=%d ld=%d", rows,
             vocab, ld);
  const int n_chunks = (vocab + SM_CHUNK - 1) / SM_CHUNK;
  TK_REQUIRE(n_chunks <= SM_MAX_CHUNKS, "sample_static: a vocabulary of %d is larger than %d", vocab,
             SM_MAX_CHUNKS * SM_CHUNK);
  TK_REQUIRE((long)rows * n_chunks <= TK_SAMPLE_STATIC_ITEMS,
             "sample_static: %d rows of %d chunks need %ld partial results, the static scratch holds %d; "
             "use tk_sample with a workspace for inputs this large",
             rows, n_chunks, (long)rows * n_chunks, TK_SAMPLE_STATIC_ITEMS);
  if (rows == 0) return 0;
  uint32_t* base = static_scratch();
  if (base == nullptr) return -3;
  // every (row, chunk) entry that the second kernel reads is written by the first: nothing to clear
  float* part_max = (float*)base;
  float* part_sum = (float*)(base + TK_SAMPLE_STATIC_ITEMS);
  int* part_arg = (int*)(base + 2 * TK_SAMPLE_STATIC_ITEMS);
  return launch_sample(logits, ld, rows, vocab, temperature, uniform, slots, last_token, out_ids, out_logprobs,
                       part_max, part_sum, part_arg, n_chunks, stream);
}

// ---------------------------------------------------------------------------
// The k most probable tokens of every row and their log-probabilities under
// softmax(logits / T) (T treated as 1 when 0), most probable first; among equal
// logits the lower index first.  Two kernels, cut like the sampler's:
//   topk_partial: one workgroup per (row, chunk): the chunk's k best in order, its
//                 maximum and sum exp((x - max) / T);
//   topk_finish:  one workgroup per row: the k best among the chunks' candidates.
// Each of the k places is one arg-max over what comes after the place before it in
// the order (value descending, index ascending): k is small, the candidates are few.
#define TOPK_MAX 32

struct Ranked {
  float v;
  int i;
};

// a stands before b in the order of the result
__device__ __forceinline__ bool before(const Ranked& a, const Ranked& b) {
  return a.v > b.v || (a.v == b.v && a.i < b.i);
}

// what is left when nothing more is eligible: it stands behind every real element
__device__ __forceinline__ Ranked nothing() { return Ranked{-INFINITY, 0x7fffffff}; }

// the first in the order over the workgroup; every thread gets it
__device__ __forceinline__ Ranked block_first(Ranked mine, Ranked* red) {
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE;
#pragma unroll
  for (int o = TK_WAVE / 2; o > 0; o >>= 1) {
    Ranked other{__shfl_xor(mine.v, o, TK_WAVE), __shfl_xor(mine.i, o, TK_WAVE)};
    if (before(other, mine)) mine = other;
  }
  __syncthreads();  // the round before has read red
  if (lane == 0) red[wave] = mine;
  __syncthreads();
  Ranked best = red[0];
  for (int w = 1; w < SM_THREADS / TK_WAVE; ++w)
    if (before(red[w], best)) best = red[w];
  return best;
}

__global__ __launch_bounds__(SM_THREADS) void topk_partial_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature, int k,
    float* __restrict__ part_val, int* __restrict__ part_idx, float* __restrict__ part_max,
    float* __restrict__ part_sum, int n_chunks) {
  __shared__ Ranked red[SM_THREADS / TK_WAVE];
  __shared__ float red_f[16];
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row];
  const float inv_t = T > 0.f ? 1.0f / T : 1.0f;
  const int begin = chunk * SM_CHUNK + tid * SM_PER_THREAD;
  Ranked held[SM_PER_THREAD];
#pragma unroll
  for (int i = 0; i < SM_PER_THREAD; ++i)
    held[i] = begin + i < vocab ? Ranked{x[begin + i], begin + i} : nothing();
  const size_t o = (size_t)row * n_chunks + chunk;
  Ranked prev{INFINITY, -1};
  float chunk_max = -INFINITY;
  for (int r = 0; r < k; ++r) {
    Ranked mine = nothing();
#pragma unroll
    for (int i = 0; i < SM_PER_THREAD; ++i)
      if (before(prev, held[i]) && before(held[i], mine)) mine = held[i];
    prev = block_first(mine, red);
    if (r == 0) chunk_max = prev.v;
    if (tid == 0) {
      part_val[o * k + r] = prev.v;
      part_idx[o * k + r] = prev.i;
    }
  }
  float local = 0.f;
#pragma unroll
  for (int i = 0; i < SM_PER_THREAD; ++i)
    local += (held[i].v == -INFINITY) ? 0.f : expf((held[i].v - chunk_max) * inv_t);
  const float total = block_sum(local, red_f);
  if (tid == 0) {
    part_max[o] = chunk_max;
    part_sum[o] = total;
  }
}

__global__ __launch_bounds__(SM_THREADS) void topk_finish_kernel(
    const float* __restrict__ temperature, int k, const float* __restrict__ part_val,
    const int* __restrict__ part_idx, const float* __restrict__ part_max,
    const float* __restrict__ part_sum, int n_chunks, int* __restrict__ out_ids,
    float* __restrict__ out_logprobs) {
  __shared__ Ranked red[SM_THREADS / TK_WAVE];
  __shared__ float red_f[16];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float T = temperature[row];
  const float inv_t = T > 0.f ? 1.0f / T : 1.0f;
  const float* pm = part_max + (size_t)row * n_chunks;
  const float* ps = part_sum + (size_t)row * n_chunks;
  const float* pv = part_val + (size_t)row * n_chunks * k;
  const int* pi = part_idx + (size_t)row * n_chunks * k;
  const int n = n_chunks * k;
  float m = -INFINITY;
  for (int c = tid; c < n_chunks; c += SM_THREADS) m = fmaxf(m, pm[c]);
  const float row_max = block_max(m, red_f);
  float mass = 0.f;
  for (int c = tid; c < n_chunks; c += SM_THREADS)
    mass += (pm[c] == -INFINITY) ? 0.f : ps[c] * expf((pm[c] - row_max) * inv_t);
  const float log_total = logf(block_sum(mass, red_f));
  Ranked prev{INFINITY, -1};
  for (int r = 0; r < k; ++r) {
    Ranked mine = nothing();
    for (int c = tid; c < n; c += SM_THREADS) {
      const Ranked cand{pv[c], pi[c]};
      if (before(prev, cand) && before(cand, mine)) mine = cand;
    }
    prev = block_first(mine, red);
    if (tid == 0) {
      out_ids[(size_t)row * k + r] = prev.i;
      out_logprobs[(size_t)row * k + r] = (prev.v - row_max) * inv_t - log_total;
    }
  }
}

// part_val and part_idx hold rows * tk_sample_chunks(vocab) * k entries, part_max and part_sum
// rows * tk_sample_chunks(vocab); out_ids and out_logprobs are [rows, k].
TK_API int tk_topk_logprobs(const float* logits, int ld, int rows, int vocab, const float* temperature,
                            int k, int* out_ids, float* out_logprobs, float* part_val, int* part_idx,
                            float* part_max, float* part_sum, hipStream_t stream) {
  TK_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "topk_logprobs: bad sizes rows=%d vocab=%d ld=%d",
             rows, vocab, ld);
  TK_REQUIRE(k >= 1 && k <= TOPK_MAX && k <= vocab,
             "topk_logprobs: k=%d is not between 1 and %d (and at most the vocabulary of %d)", k,
             TOPK_MAX, vocab);
  const int n_chunks = (vocab + SM_CHUNK - 1) / SM_CHUNK;
  TK_REQUIRE(n_chunks <= SM_MAX_CHUNKS, "topk_logprobs: a vocabulary of %d is larger than %d", vocab,
             SM_MAX_CHUNKS * SM_CHUNK);
  TK_REQUIRE(rows < 65536, "topk_logprobs: %d rows are too many for one call", rows);
  TK_REQUIRE(part_val && part_idx && part_max && part_sum, "topk_logprobs: scratch missing");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(topk_partial_kernel, dim3(n_chunks, rows), dim3(SM_THREADS), 0, stream, logits,
                     ld, vocab, temperature, k, part_val, part_idx, part_max, part_sum, n_chunks);
  TK_CHECK_LAUNCH("topk_partial");
  hipLaunchKernelGGL(topk_finish_kernel, dim3(rows), dim3(SM_THREADS), 0, stream, temperature, k,
                     part_val, part_idx, part_max, part_sum, n_chunks, out_ids, out_logprobs);
  TK_CHECK_LAUNCH("topk_finish");
  return 0;
}
