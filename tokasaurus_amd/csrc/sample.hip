// Sampling from 32-bit logits, one workgroup per row:
//   temperature == 0: the index of the largest raw logit (the lowest index on a tie);
//   temperature  > 0: p = softmax(logits / T) and the smallest index whose
//                     cumulative probability exceeds the row's uniform number u.
// Also the chosen token's log-probability under p (T treated as 1 when 0), and
// optionally the token written to the request's slot for the next step's embedding.
#include "common.h"

#define SM_THREADS 1024

__global__ __launch_bounds__(SM_THREADS) void sample_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
    const float* __restrict__ uniform, const int* __restrict__ slots, int* __restrict__ last_token,
    int* __restrict__ out_ids, float* __restrict__ out_logprobs) {
  __shared__ float red[16];
  __shared__ float wave_tot[16];
  __shared__ int red_i[16];
  __shared__ int chosen;
  __shared__ float cum[SM_THREADS];
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & (TK_WAVE - 1), wave = tid / TK_WAVE;
  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row];
  const float inv_t = T > 0.f ? 1.0f / T : 1.0f;

  // contiguous segment of this thread
  const int per = (vocab + SM_THREADS - 1) / SM_THREADS;
  const int begin = min(tid * per, vocab), end = min(begin + per, vocab);

  // maximum and its first index
  float best = -INFINITY;
  int best_i = vocab;
  for (int i = begin; i < end; ++i) {
    const float v = x[i];
    if (v > best) { best = v; best_i = i; }
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
  __syncthreads();
  const float row_max = m;
  const int argmax = mi;

  // sum of exp((x - max) / T): per thread, then per wave, then the whole row
  float local = 0.f;
  for (int i = begin; i < end; ++i) local += expf((x[i] - row_max) * inv_t);
  // inclusive scan inside the wavefront (segments are ordered by thread id)
  float scan = local;
#pragma unroll
  for (int o = 1; o < TK_WAVE; o <<= 1) {
    const float up = __shfl_up(scan, o, TK_WAVE);
    if (lane >= o) scan += up;
  }
  if (lane == TK_WAVE - 1) wave_tot[wave] = scan;
  __syncthreads();
  float before = 0.f, total = 0.f;
  for (int w = 0; w < SM_THREADS / TK_WAVE; ++w) {
    if (w < wave) before += wave_tot[w];
    total += wave_tot[w];
  }
  // cum[i]: mass of the segments of threads 0..i.  Thread i owns the interval
  // [cum[i-1], cum[i]); the intervals tile [0, cum[last]) without gaps.
  cum[tid] = before + scan;
  if (tid == 0) chosen = (T > 0.f) ? vocab - 1 : argmax;
  __syncthreads();
  if (T > 0.f) {
    const float target = uniform[row] * total;
    const float lower = tid > 0 ? cum[tid - 1] : 0.f;
    if (lower <= target && target < cum[tid] && begin < end) {
      float c = lower;
      int pick = end - 1;
      for (int i = begin; i < end; ++i) {
        c += expf((x[i] - row_max) * inv_t);
        if (c > target) { pick = i; break; }
      }
      atomicMin(&chosen, pick);
    }
  }
  __syncthreads();
  if (tid == 0) {
    const int id = chosen;
    out_ids[row] = id;
    if (out_logprobs) out_logprobs[row] = (x[id] - row_max) * inv_t - logf(total);
    if (last_token && slots) last_token[slots[row]] = id;
  }
}

extern "C" int tk_sample(const float* logits, int ld, int rows, int vocab, const float* temperature,
                         const float* uniform, const int* slots, int* last_token, int* out_ids,
                         float* out_logprobs, hipStream_t stream) {
  TK_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d vocab=%d ld=%d", rows,
             vocab, ld);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SM_THREADS), 0, stream, logits, ld, vocab,
                     temperature, uniform, slots, last_token, out_ids, out_logprobs);
  TK_CHECK_LAUNCH("sample");
  return 0;
}
