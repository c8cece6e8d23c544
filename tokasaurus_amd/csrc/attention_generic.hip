// Paged attention for any head size, group size, page size and window, in
// 32-bit arithmetic: the attention of the true 32-bit path, and of the bfloat16
// path for shapes the MFMA kernels refuse.
//
// One workgroup per (query token, kv head).  It serves the `group` query heads
// that share the kv head, walks the token's keys in chunks of CH positions
// aligned to absolute multiples of CH (so the order of the reduction depends
// only on the token's own position, never on the batch), and keeps a running
// maximum, sum and weighted value sum per query head (online softmax).
//
//   K pages: [page][kv head][d / 8][P][8]   V pages: [page][kv head][P / 4][d][4]
//   (key_offset and value_offset of common.h); block_table[req][pos / P] is the page of a position.
// A query at position p sees positions max(0, p - window + 1) .. p (window <= 0: all).
#include "common.h"

#define AG_THREADS 256
#define AG_MAX_ACC 8  // outputs per thread: group * d <= AG_THREADS * AG_MAX_ACC

template <typename T, int CH>
__global__ __launch_bounds__(AG_THREADS) void paged_attention_generic_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
    const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ token_req,
    const int* __restrict__ positions, int nq, int nkv, int d, int P, int window, float scale) {
  extern __shared__ float smem[];
  const int t = blockIdx.x, g = blockIdx.y;
  const int group = nq / nkv;
  const int tid = threadIdx.x;
  const int lane = tid & (TK_WAVE - 1), wave = tid / TK_WAVE;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int* table = block_table + (size_t)token_req[t] * table_stride;

  float* qs = smem;                    // [group][d]
  float* Ks = qs + group * d;          // [CH][d + 1]
  float* Vs = Ks + CH * (d + 1);       // [CH][d]
  float* Ss = Vs + CH * d;             // [group][CH]
  float* st_m = Ss + group * CH;       // [group] running maximum
  float* st_l = st_m + group;          // [group] running sum
  float* st_a = st_l + group;          // [group] rescale factor of this chunk

  const int n_out = group * d;
  for (int i = tid; i < n_out; i += AG_THREADS)
    qs[i] = to_f32<T>(q[(size_t)t * q_stride + (size_t)g * group * d + i]);
  if (tid < group) {
    st_m[tid] = -INFINITY;
    st_l[tid] = 0.f;
  }
  float acc[AG_MAX_ACC];
#pragma unroll
  for (int r = 0; r < AG_MAX_ACC; ++r) acc[r] = 0.f;

  for (int c0 = (lo / CH) * CH; c0 <= pos; c0 += CH) {
    __syncthreads();  // the chunk before is consumed; qs and stats are written
    // stage the chunk's keys and values as 32-bit values
    for (int i = tid; i < CH * d; i += AG_THREADS) {
      const int j = i / d, e = i % d;
      const int kp = c0 + j;
      float kv = 0.f, vv = 0.f;
      if (kp >= lo && kp <= pos) {
        const int page = table[kp / P];
        const int p = kp % P;
        const size_t base = ((size_t)page * nkv + g) * P * d;
        kv = to_f32<T>(kcache[base + key_offset(P, p, e)]);
        vv = to_f32<T>(vcache[base + value_offset(d, p, e)]);
      }
      Ks[j * (d + 1) + e] = kv;
      Vs[j * d + e] = vv;
    }
    __syncthreads();
    // scores
    for (int i = tid; i < group * CH; i += AG_THREADS) {
      const int gq = i / CH, j = i % CH;
      const int kp = c0 + j;
      float s = -INFINITY;
      if (kp >= lo && kp <= pos) {
        float dot = 0.f;
        const float* qv = qs + gq * d;
        const float* kv = Ks + j * (d + 1);
        for (int e = 0; e < d; ++e) dot = fmaf(qv[e], kv[e], dot);
        s = dot * scale;
      }
      Ss[i] = s;
    }
    __syncthreads();
    // softmax bookkeeping: one wavefront per query head, one position per lane
    for (int gq = wave; gq < group; gq += AG_THREADS / TK_WAVE) {
      const float s = lane < CH ? Ss[gq * CH + lane] : -INFINITY;
      const float m_old = st_m[gq];
      const float m_new = fmaxf(m_old, wave_max(s));
      const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
      const float psum = wave_sum(p);
      if (lane < CH) Ss[gq * CH + lane] = p;
      if (lane == 0) {
        const float alpha = (m_old == -INFINITY) ? 0.f : expf(m_old - m_new);
        st_m[gq] = m_new;
        st_l[gq] = st_l[gq] * alpha + psum;
        st_a[gq] = alpha;
      }
    }
    __syncthreads();
    // weighted values
#pragma unroll
    for (int r = 0; r < AG_MAX_ACC; ++r) {
      const int i = tid + r * AG_THREADS;
      if (i < n_out) {
        const int gq = i / d, e = i % d;
        float a = acc[r] * st_a[gq];
        const float* pv = Ss + gq * CH;
        for (int j = 0; j < CH; ++j) a = fmaf(pv[j], Vs[j * d + e], a);
        acc[r] = a;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < AG_MAX_ACC; ++r) {
    const int i = tid + r * AG_THREADS;
    if (i < n_out) {
      const int gq = i / d;
      out[(size_t)t * out_stride + (size_t)g * group * d + i] = from_f32<T>(acc[r] / st_l[gq]);
    }
  }
}

static size_t ag_smem_bytes(int group, int d, int ch) {
  return sizeof(float) * ((size_t)group * d + (size_t)ch * (d + 1) + (size_t)ch * d +
                          (size_t)group * ch + 3 * (size_t)group);
}

template <typename T, int CH>
static void ag_launch(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                      const void* vcache, const int* block_table, int table_stride,
                      const int* token_req, const int* positions, int n_tokens, int nq, int nkv,
                      int d, int P, int window, float scale, hipStream_t stream) {
  hipLaunchKernelGGL((paged_attention_generic_kernel<T, CH>), dim3(n_tokens, nkv),
                     dim3(AG_THREADS), ag_smem_bytes(nq / nkv, d, CH), stream, (const T*)q,
                     q_stride, (T*)out, out_stride, (const T*)kcache, (const T*)vcache,
                     block_table, table_stride, token_req, positions, nq, nkv, d, P, window, scale);
}

// Whether the kernel takes this group and head size at all (0 and the reason in tk_last_error
// when not): asked when a cache is made, so that a model is refused before its first step.
TK_API int tk_paged_attention_generic_fits(int nq, int nkv, int d) {
  TK_REQUIRE(nq > 0 && nkv > 0 && d > 0 && nq % nkv == 0, "paged_attention: bad sizes nq=%d nkv=%d d=%d", nq, nkv, d);
  const int group = nq / nkv;
  TK_REQUIRE(group * d <= AG_THREADS * AG_MAX_ACC,
             "paged_attention: group %d x head size %d exceeds %d outputs per kv head", group, d,
             AG_THREADS * AG_MAX_ACC);
  TK_REQUIRE(ag_smem_bytes(group, d, 8) <= 64 * 1024,
             "paged_attention: head size %d with group %d does not fit the local memory", d, group);
  return 0;
}

TK_API int tk_paged_attention_generic(int dt, const void* q, int q_stride, void* out,
                                          int out_stride, const void* kcache, const void* vcache,
                                          const int* block_table, int table_stride,
                                          const int* token_req, const int* positions, int n_tokens,
                                          int nq, int nkv, int d, int P, int window, float scale,
                                          hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && nq > 0 && nkv > 0 && d > 0 && P > 0 && nq % nkv == 0,
             "paged_attention: bad sizes tokens=%d nq=%d nkv=%d d=%d P=%d", n_tokens, nq, nkv, d,
             P);
  const int group = nq / nkv;
  TK_REQUIRE(group * d <= AG_THREADS * AG_MAX_ACC,
             "paged_attention: group %d x head size %d exceeds %d outputs per kv head", group, d,
             AG_THREADS * AG_MAX_ACC);
  TK_REQUIRE(q_stride >= nq * d && out_stride >= nq * d, "paged_attention: row strides too short");
  TK_REQUIRE(nkv < 65536, "paged_attention: too many kv heads");
  if (n_tokens == 0) return 0;
  const size_t limit = 64 * 1024;
  int ch = 64;
  while (ch > 8 && ag_smem_bytes(group, d, ch) > limit) ch /= 2;
  TK_REQUIRE(ag_smem_bytes(group, d, ch) <= limit,
             "paged_attention: head size %d with group %d does not fit the local memory", d, group);
#define AG_CASE(T, CHV)                                                                         \
  ag_launch<T, CHV>(q, q_stride, out, out_stride, kcache, vcache, block_table, table_stride,    \
                    token_req, positions, n_tokens, nq, nkv, d, P, window, scale, stream)
  if (dt == TK_F32) {
    if (ch == 64) AG_CASE(float, 64);
    else if (ch == 32) AG_CASE(float, 32);
    else if (ch == 16) AG_CASE(float, 16);
    else AG_CASE(float, 8);
  } else {
    if (ch == 64) AG_CASE(bf16_t, 64);
    else if (ch == 32) AG_CASE(bf16_t, 32);
    else if (ch == 16) AG_CASE(bf16_t, 16);
    else AG_CASE(bf16_t, 8);
  }
#undef AG_CASE
  TK_CHECK_LAUNCH("paged_attention_generic");
  return 0;
}
