// bfloat16 matrix products for few rows (decode):  C[M,N] = A[M,K] * W[N,K]^T, M <= 128,
// on the gfx950 matrix cores with 32-bit accumulation, an optional RMSNorm of A fused
// in front and an epilogue fused behind.
//
// The product is bound by reading W once.  Weight rows are cut into tiles of 16;
// lane l of a wavefront streams the 8 values W[row l%16][32*step + 8*(l/16) .. +8]
// of a tile straight from memory into the first operand of v_mfma_f32_16x16x32_bf16
// (a row is read 64 contiguous bytes at a time); up to 16 tokens are the second
// operand, so
//     acc[j] of lane (r = l%16, q = l/16)  =  C[token 16*mb + r][row 16*tile + 4*q + j].
// No workgroup talks to another and partial sums inside a workgroup are added in
// wavefront order through LDS, so every output has one fixed order of summation.
//
// Two kernels:
//   gemm_skinny_kernel (M <= 16, or any M as the fallback): a workgroup owns NT tiles
//     and all of K; its wavefronts split K and read A straight from memory.
//   gemm_staged_kernel (16 < M <= 128): a workgroup is 4 x WK wavefronts; the 4
//     wavefronts of a row own NT tiles each and share the K range of their row, whose
//     part of A passes through LDS (double buffered, 4 steps of 32 a round) so that A
//     is read from the caches once per workgroup and not once per wavefront.
//
// Norm in front (norm_w != null): the product of RMSNorm(A) is rstd[row] * ((A * w) W^T),
// so the kernel multiplies A by the norm weight on the way in (rounded to bfloat16
// once), sums the squares of the A values it reads anyway in 32-bit, and scales each
// output row by rstd = 1 / sqrt(mean(A^2) + eps) in the epilogue: no pass over A of its
// own and no wait in front of the weight stream.  Epilogues: plain store, + residual,
// SwiGLU (the wavefront takes the same 16 rows of the gate and of the up projection),
// 32-bit store.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2, EPI_F32 = 3 };

struct GemmArgs {
  const bf16_t* A;
  int lda;
  const bf16_t* W;
  void* C;
  int ldc;
  const bf16_t* residual;
  int ldr;
  const void* norm_w;  // [K] bfloat16, or float when norm_w_f32
  int norm_w_f32;
  float eps;
  int M, N, K;  // N: outputs (for SwiGLU the intermediate size; W then has 2N rows, gate first)
  int TH;       // weight rows of a tile that are used (16, or 8 to make twice the workgroups of a narrow output)
};

__device__ __forceinline__ float silu_mul_bf16(float g, float u) {
  const float gr = round_to<bf16_t>(g), ur = round_to<bf16_t>(u);
  const float s = round_to<bf16_t>(gr / (1.0f + expf(-gr)));
  return s * ur;
}

template <int EPI>
__device__ __forceinline__ void store4(const GemmArgs& a, f32x4_t v, f32x4_t up, float scale, int token, int n) {
  if (token >= a.M) return;
  float o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    o[j] = v[j] * scale;
    if (EPI == EPI_SWIGLU) o[j] = silu_mul_bf16(v[j] * scale, up[j] * scale);
    if (EPI == EPI_RESIDUAL && n + j < a.N)
      o[j] = round_to<bf16_t>(o[j]) + __bfloat162float(a.residual[(size_t)token * a.ldr + n + j]);
  }
  if (EPI == EPI_F32) {
    float* c = (float*)a.C + (size_t)token * a.ldc + n;
    if (n + 3 < a.N && (a.ldc & 3) == 0) {
      *(f32x4_t*)c = f32x4_t{o[0], o[1], o[2], o[3]};
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < a.N) c[j] = o[j];
    }
  } else {
    bf16_t* c = (bf16_t*)a.C + (size_t)token * a.ldc + n;
    if (n + 3 < a.N && (a.ldc & 3) == 0) {
      union { bf16_t h[4]; uint2 u; } pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) pk.h[j] = __float2bfloat16(o[j]);
      *(uint2*)c = pk.u;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < a.N) c[j] = __float2bfloat16(o[j]);
    }
  }
}

__device__ __forceinline__ bf16x8_t zero8() {
  bf16x8_t z;
#pragma unroll
  for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.f;
  return z;
}

// 8 values of a row times the norm weight, rounded once; their squares are added to `ss`.
__device__ __forceinline__ bf16x8_t weigh_piece(bf16x8_t x, const void* w, int w_f32, int k, float& ss) {
  bf16x8_t o;
  if (w_f32) {
    const float* wf = (const float*)w + k;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float xe = (float)x[e];
      ss = fmaf(xe, xe, ss);
      o[e] = (__bf16)(wf[e] * xe);
    }
  } else {
    const bf16x8_t wv = *(const bf16x8_t*)((const bf16_t*)w + k);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float xe = (float)x[e];
      ss = fmaf(xe, xe, ss);
      o[e] = (__bf16)((float)wv[e] * xe);
    }
  }
  return o;
}

#define SK_MAX_WAVES 16

// LDS of the skinny kernel: [sums: waves * NT * MB * 64 f32x4][squares: waves * 16 * MB floats]
template <int MB, int NT, int EPI, bool NORM>
__global__ __launch_bounds__(SK_MAX_WAVES * 64) void gemm_skinny_kernel(GemmArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int U = (NT + MB <= 3) ? 8 : ((NT + MB <= 6) ? 4 : 2);  // steps whose loads are in flight together
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int WK = blockDim.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int g = blockIdx.x;
  const int K32 = (a.K + 31) >> 5;
  const int ks0 = (int)((long)K32 * wave / WK), ks1 = (int)((long)K32 * (wave + 1) / WK);
  const bool k_exact = (a.K & 31) == 0;
  f32x4_t* red = (f32x4_t*)smem;
  float* sq = (float*)(red + (WK > 1 ? (size_t)WK * NT * MB * 64 : 0));

  // rows of W this lane streams (clamped: rows past the end are masked at the store);
  // with tiles of 8 rows the upper lanes have no row and hold zeros
  const int TH = a.TH;
  const bool has_row = r < TH;
  const bf16_t* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int row;
    if (EPI == EPI_SWIGLU) {
      row = min(g * TH + r, a.N - 1) + t * a.N;  // t = 0 gate, t = 1 up
    } else {
      row = min((g * NT + t) * TH + r, a.N - 1);
    }
    wp[t] = a.W + (size_t)row * a.K + q * 8;
  }
  const bf16_t* ap[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) ap[mb] = a.A + (size_t)min(mb * 16 + r, a.M - 1) * a.lda + q * 8;

  float ss[MB];  // squares of the values of row 16 mb + r that this lane has read
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) ss[mb] = 0.f;

  f32x4_t acc[NT][MB];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[t][mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  int ks = ks0;
  if (k_exact) {
    for (; ks + U <= ks1; ks += U) {
      bf16x8_t w[U][NT], av[U][MB];
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          if (has_row) {
            w[u][t] = *(const bf16x8_t*)(wp[t] + (size_t)(ks + u) * 32);
          } else {
            w[u][t] = zero8();
          }
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) av[u][mb] = *(const bf16x8_t*)(ap[mb] + (size_t)(ks + u) * 32);
      }
      if (NORM) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            av[u][mb] = weigh_piece(av[u][mb], a.norm_w, a.norm_w_f32, (ks + u) * 32 + q * 8, ss[mb]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][t], av[u][mb], acc[t][mb], 0, 0, 0);
    }
  }
  for (; ks < ks1; ++ks) {
    // a step may reach past K (K is a multiple of 8): read a valid chunk and zero the weight
    const bool k_ok = ks * 32 + q * 8 < a.K;
    const long off = k_ok ? (long)ks * 32 : -(long)(q * 8);
    bf16x8_t w[NT], av[MB];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      w[t] = *(const bf16x8_t*)(wp[t] + off);
      if (!k_ok || !has_row) w[t] = zero8();
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      av[mb] = *(const bf16x8_t*)(ap[mb] + off);
      if (NORM && k_ok) av[mb] = weigh_piece(av[mb], a.norm_w, a.norm_w_f32, ks * 32 + q * 8, ss[mb]);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[t], av[mb], acc[t][mb], 0, 0, 0);
  }

  if (NORM) {
    // the row's squares over this wavefront's part of K: every lane of the row gets the sum
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      ss[mb] += __shfl_xor(ss[mb], 16, 64);
      ss[mb] += __shfl_xor(ss[mb], 32, 64);
    }
  }
  // add the wavefronts' partial sums in wavefront order
  if (WK > 1) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) red[(wave * NT * MB + t * MB + mb) * 64 + lane] = acc[t][mb];
    if (NORM && q == 0) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) sq[wave * 16 * MB + mb * 16 + r] = ss[mb];
    }
    __syncthreads();
  }
  constexpr int UNITS = (EPI == EPI_SWIGLU ? 1 : NT) * MB * 64;
  for (int u = tid; u < UNITS; u += blockDim.x) {
    const int l = u & 63, mb = (u >> 6) % MB, t = (u >> 6) / MB;
    const int token = mb * 16 + (l & 15), qq = l >> 4;
    f32x4_t s0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, s1 = s0;
    float total = 0.f;
    if (WK > 1) {
      for (int w = 0; w < WK; ++w) {
        s0 += red[(w * NT * MB + t * MB + mb) * 64 + l];
        if (EPI == EPI_SWIGLU) s1 += red[(w * NT * MB + MB + mb) * 64 + l];
        if (NORM) total += sq[w * 16 * MB + mb * 16 + (l & 15)];
      }
    } else {
      // one wavefront: unit u is this very lane's accumulator (u < 64 * NT * MB, tid == lane)
#pragma unroll
      for (int tt = 0; tt < NT; ++tt)
#pragma unroll
        for (int mm = 0; mm < MB; ++mm) {
          if (tt == t && mm == mb) s0 = acc[tt][mm];
          if (EPI == EPI_SWIGLU && tt == 1 && mm == mb) s1 = acc[tt][mm];
          if (NORM && mm == mb) total = ss[mm];
        }
    }
    if (qq * 4 >= TH) continue;
    const float scale = NORM ? 1.0f / sqrtf(total / (float)a.K + a.eps) : 1.0f;
    const int n = (EPI == EPI_SWIGLU ? g : g * NT + t) * TH + qq * 4;
    store4<EPI>(a, s0, s1, scale, token, n);
  }
}

// ---------------------------------------------------------------------------------
// 16 < M <= 128: A passes through LDS.
// A workgroup is 4 x WK wavefronts; wavefront (wn, wk) owns the NT tiles of index
// (4 * workgroup + wn) * NT + t and the steps of K that row wk of the workgroup has.
// A round is 4 steps; wavefront wn of a row brings step wn of the round into LDS in
// the lane order of the matrix-core operand (one KB a unit), for all MB blocks of 16
// tokens, while the round before is multiplied.
// LDS: [squares: waves * 16 * MB floats][2 buffers x WK x 4 steps x MB units of 1 KB],
// the sums of the wavefront rows reuse the buffers after the last round.
// ---------------------------------------------------------------------------------
#define ST_WN 4
#define ST_SC 4

template <int MB, int NT, int EPI, bool NORM>
__global__ __launch_bounds__(1024) void gemm_staged_kernel(GemmArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int nwaves = blockDim.x >> 6;
  const int WK = nwaves / ST_WN;
  const int wn = wave % ST_WN, wk = wave / ST_WN;
  const int r = lane & 15, q = lane >> 4;
  const int K32 = (a.K + 31) >> 5;
  const int ks0 = (int)((long)K32 * wk / WK), ks1 = (int)((long)K32 * (wk + 1) / WK);
  const int rounds = ((K32 + WK - 1) / WK + ST_SC - 1) / ST_SC;
  float* sq = (float*)smem;  // [wave][16 * MB]
  unsigned char* stage = smem + (NORM ? (size_t)nwaves * 16 * MB * sizeof(float) : 0);
  bf16x8_t* stage_v = (bf16x8_t*)stage;  // [buffer][wk][step][mb][lane]
  f32x4_t* red = (f32x4_t*)stage;         // [wk][wn][NT * MB][lane], after the last round

  const int unit = blockIdx.x * ST_WN + wn;  // SwiGLU: a pair of tiles; else NT tiles
  const bf16_t* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int row;
    if (EPI == EPI_SWIGLU) {
      row = min(unit * 16 + r, a.N - 1) + t * a.N;
    } else {
      row = min((unit * NT + t) * 16 + r, a.N - 1);
    }
    wp[t] = a.W + (size_t)row * a.K + q * 8;
  }
  const bf16_t* ap[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) ap[mb] = a.A + (size_t)min(mb * 16 + r, a.M - 1) * a.lda + q * 8;

  float ss[MB];  // squares of the values of row 16 mb + r that this lane has brought in
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) ss[mb] = 0.f;

  // this wavefront's step of a round of A, for every block of tokens
  auto load_a = [&](int round, bf16x8_t (&piece)[MB]) {
    const int s = ks0 + round * ST_SC + wn;
    const int k = s * 32 + q * 8;
    const bool ok = s < ks1 && k < a.K;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      if (ok) {
        piece[mb] = *(const bf16x8_t*)(ap[mb] + (size_t)s * 32);
        if (NORM) piece[mb] = weigh_piece(piece[mb], a.norm_w, a.norm_w_f32, k, ss[mb]);
      } else {
        piece[mb] = zero8();
      }
    }
  };
  auto store_a = [&](int buf, const bf16x8_t (&piece)[MB]) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      stage_v[((((size_t)buf * WK + wk) * ST_SC + wn) * MB + mb) * 64 + lane] = piece[mb];
  };
  auto load_w = [&](int round, bf16x8_t (&w)[ST_SC][NT]) {
#pragma unroll
    for (int j = 0; j < ST_SC; ++j) {
      const int s = ks0 + round * ST_SC + j;
      const bool ok = s < ks1 && s * 32 + q * 8 < a.K;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (ok) {
          w[j][t] = *(const bf16x8_t*)(wp[t] + (size_t)s * 32);
        } else {
          w[j][t] = zero8();
        }
      }
    }
  };

  f32x4_t acc[NT][MB];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[t][mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  bf16x8_t w_cur[ST_SC][NT], piece[MB];
  load_w(0, w_cur);
  load_a(0, piece);
  store_a(0, piece);
  __syncthreads();
  int buf = 0;
  for (int round = 0; round < rounds; ++round) {
    bf16x8_t w_nxt[ST_SC][NT];
    const bool more = round + 1 < rounds;
    if (more) {
      load_w(round + 1, w_nxt);
      load_a(round + 1, piece);
    }
#pragma unroll
    for (int j = 0; j < ST_SC; ++j) {
      // steps past this row's range carry zero weights: their product adds nothing
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const bf16x8_t av = stage_v[((((size_t)buf * WK + wk) * ST_SC + j) * MB + mb) * 64 + lane];
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[j][t], av, acc[t][mb], 0, 0, 0);
      }
    }
    if (more) {
      store_a(buf ^ 1, piece);
#pragma unroll
      for (int j = 0; j < ST_SC; ++j)
#pragma unroll
        for (int t = 0; t < NT; ++t) w_cur[j][t] = w_nxt[j][t];
    }
    __syncthreads();
    buf ^= 1;
  }

  // every piece of A was brought in by one wavefront: the squares of a row are the sum over all
  if (NORM) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      ss[mb] += __shfl_xor(ss[mb], 16, 64);
      ss[mb] += __shfl_xor(ss[mb], 32, 64);
      if (q == 0) sq[wave * 16 * MB + mb * 16 + r] = ss[mb];
    }
  }
  // add the rows' partial sums in row order
  if (WK > 1) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) red[((size_t)(wk * ST_WN + wn) * NT * MB + t * MB + mb) * 64 + lane] = acc[t][mb];
  }
  if (WK > 1 || NORM) __syncthreads();
  constexpr int TN = (EPI == EPI_SWIGLU ? 1 : NT);
  if (WK == 1) {
    // every wavefront stores its own sums
    const int token0 = lane & 15, qq = lane >> 4;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      float total = 0.f;
      if (NORM)
        for (int w = 0; w < nwaves; ++w) total += sq[w * 16 * MB + mb * 16 + token0];
      const float scale = NORM ? 1.0f / sqrtf(total / (float)a.K + a.eps) : 1.0f;
#pragma unroll
      for (int t = 0; t < TN; ++t) {
        const int n = (EPI == EPI_SWIGLU ? unit : unit * NT + t) * 16 + qq * 4;
        store4<EPI>(a, acc[t][mb], acc[NT - 1][mb], scale, mb * 16 + token0, n);
      }
    }
    return;
  }
  constexpr int UNITS = ST_WN * TN * MB * 64;
  for (int u = tid; u < UNITS; u += blockDim.x) {
    const int l = u & 63;
    int rest = u >> 6;
    const int mb = rest % MB;
    rest /= MB;
    const int t = rest % TN, own = rest / TN;
    const int token = mb * 16 + (l & 15), qq = l >> 4;
    f32x4_t s0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, s1 = s0;
    for (int w = 0; w < WK; ++w) {
      s0 += red[((size_t)(w * ST_WN + own) * NT * MB + t * MB + mb) * 64 + l];
      if (EPI == EPI_SWIGLU) s1 += red[((size_t)(w * ST_WN + own) * NT * MB + MB + mb) * 64 + l];
    }
    float total = 0.f;
    if (NORM)
      for (int w = 0; w < nwaves; ++w) total += sq[w * 16 * MB + mb * 16 + (l & 15)];
    const float scale = NORM ? 1.0f / sqrtf(total / (float)a.K + a.eps) : 1.0f;
    const int tile_group = blockIdx.x * ST_WN + own;
    const int n = (EPI == EPI_SWIGLU ? tile_group : tile_group * NT + t) * 16 + qq * 4;
    store4<EPI>(a, s0, s1, scale, token, n);
  }
}

// ---------------------------------------------------------------------------------
// launch
// ---------------------------------------------------------------------------------
template <typename Kernel>
static bool allow_lds(Kernel kernel, size_t lds) {
  if (lds <= 64 * 1024) return true;
  return hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess;
}

template <int MB, int NT, int EPI, bool NORM>
static bool launch_skinny_one(const GemmArgs& a, int groups, int WK, hipStream_t stream) {
  size_t lds = WK > 1 ? (size_t)WK * NT * MB * 64 * sizeof(f32x4_t) : 0;
  if (NORM && WK > 1) lds += (size_t)WK * 16 * MB * sizeof(float);
  auto kernel = gemm_skinny_kernel<MB, NT, EPI, NORM>;
  if (!allow_lds(kernel, lds)) return false;
  hipLaunchKernelGGL(kernel, dim3(groups), dim3(WK * 64), lds, stream, a);
  return true;
}

template <int MB, int NT, int EPI, bool NORM>
static bool launch_staged_one(const GemmArgs& a, int groups, int WK, hipStream_t stream) {
  size_t lds = (size_t)2 * WK * ST_SC * MB * 1024;
  const size_t red = WK > 1 ? (size_t)WK * ST_WN * NT * MB * 64 * sizeof(f32x4_t) : 0;
  if (red > lds) lds = red;
  if (NORM) lds += (size_t)WK * ST_WN * 16 * MB * sizeof(float);
  auto kernel = gemm_staged_kernel<MB, NT, EPI, NORM>;
  if (!allow_lds(kernel, lds)) return false;
  hipLaunchKernelGGL(kernel, dim3(groups), dim3(WK * ST_WN * 64), lds, stream, a);
  return true;
}

template <int MB, int NT, bool STAGED>
static bool launch_epi(const GemmArgs& a, int epi, bool norm, int groups, int WK, hipStream_t stream) {
#define TK_GEMM_CASE(E)                                                                         \
  if (STAGED)                                                                                   \
    return norm ? launch_staged_one<MB, NT, E, true>(a, groups, WK, stream)                     \
                : launch_staged_one<MB, NT, E, false>(a, groups, WK, stream);                   \
  else                                                                                          \
    return norm ? launch_skinny_one<MB, NT, E, true>(a, groups, WK, stream)                     \
                : launch_skinny_one<MB, NT, E, false>(a, groups, WK, stream);
  switch (epi) {
    case EPI_STORE: TK_GEMM_CASE(EPI_STORE)
    case EPI_RESIDUAL:
      if (STAGED) return launch_staged_one<MB, NT, EPI_RESIDUAL, false>(a, groups, WK, stream);
      return launch_skinny_one<MB, NT, EPI_RESIDUAL, false>(a, groups, WK, stream);
    case EPI_F32: TK_GEMM_CASE(EPI_F32)
    default: return false;
  }
#undef TK_GEMM_CASE
}

template <int MB, bool STAGED>
static bool launch_mb(const GemmArgs& a, int epi, bool norm, int NT, int groups, int WK, hipStream_t stream) {
  if (epi == EPI_SWIGLU) {
    if (STAGED)
      return norm ? launch_staged_one<MB, 2, EPI_SWIGLU, true>(a, groups, WK, stream)
                  : launch_staged_one<MB, 2, EPI_SWIGLU, false>(a, groups, WK, stream);
    return norm ? launch_skinny_one<MB, 2, EPI_SWIGLU, true>(a, groups, WK, stream)
                : launch_skinny_one<MB, 2, EPI_SWIGLU, false>(a, groups, WK, stream);
  }
  return NT == 1 ? launch_epi<MB, 1, STAGED>(a, epi, norm, groups, WK, stream)
                 : launch_epi<MB, 2, STAGED>(a, epi, norm, groups, WK, stream);
}

// A [M, K] bfloat16 (rows lda apart), W [N, K] row-major ([2N, K] gate over up for SwiGLU),
// C [M, N].  norm_w (may be null): RMSNorm weight [K] applied to A first, bfloat16 or
// float (norm_w_f32).  waves_k: wavefronts (skinny) or wavefront rows (staged) that split
// K inside a workgroup (0 = choose); tiles: weight tiles of 16 rows per wavefront, 1 or 2
// (0 = choose; SwiGLU always pairs gate and up); staged: -1 = choose, 0 = skinny, 1 = staged;
// tile_rows: weight rows of a tile that the skinny kernel uses, 16 or 8 (0 = choose).
TK_API int tk_gemm_skinny_bf16(const void* A, int lda, const void* W, void* C, int ldc,
                                   const void* residual, int ldr, const void* norm_w,
                                   int norm_w_f32, float eps, int M, int N, int K, int epi,
                                   int waves_k, int tiles, int staged, int tile_rows,
                                   hipStream_t stream) {
  TK_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
  TK_REQUIRE(M <= 128, "gemm_skinny: at most 128 rows, got %d", M);
  TK_REQUIRE(epi >= EPI_STORE && epi <= EPI_F32, "gemm_skinny: unknown epilogue %d", epi);
  TK_REQUIRE(K % 8 == 0, "gemm_skinny: K=%d must be a multiple of 8 for the bfloat16 kernels", K);
  TK_REQUIRE(lda % 8 == 0 && ((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0,
             "gemm_skinny: rows of A and W must be 16-byte aligned (lda=%d)", lda);
  TK_REQUIRE(!norm_w || ((uintptr_t)norm_w & 15) == 0, "gemm_skinny: the norm weight must be 16-byte aligned");
  TK_REQUIRE(lda >= K && ldc >= N, "gemm_skinny: strides shorter than rows");
  TK_REQUIRE(epi != EPI_RESIDUAL || (residual && ldr >= N), "gemm_skinny: residual missing or too narrow");
  if (M == 0) return 0;
  GemmArgs a;
  a.A = (const bf16_t*)A; a.lda = lda; a.W = (const bf16_t*)W; a.C = C; a.ldc = ldc;
  a.residual = (const bf16_t*)residual; a.ldr = ldr; a.norm_w = norm_w; a.norm_w_f32 = norm_w_f32;
  a.eps = eps; a.M = M; a.N = N; a.K = K; a.TH = 16;
  TK_REQUIRE(tile_rows == 0 || tile_rows == 8 || tile_rows == 16, "gemm_skinny: tile_rows %d is not 0, 8 or 16", tile_rows);
  const bool norm = norm_w != nullptr;

  const int n16 = (N + 15) / 16;
  const int MB = M <= 16 ? 1 : (M <= 32 ? 2 : (M <= 64 ? 4 : 8));
  const int K32 = (K + 31) / 32;
  const int n16_units = epi == EPI_SWIGLU ? n16 : n16;
  // measured on an MI355X: passing A through LDS pays for a wide output (the head) from 5 rows on,
  // where many wavefronts of a workgroup share it; a narrow one needs every tile in a workgroup of its own
  const bool use_staged = (staged < 0 ? M > 4 && K32 >= 2 * ST_SC && n16_units >= 2048 : staged != 0);
  TK_REQUIRE(!(norm && epi == EPI_RESIDUAL), "gemm_skinny: a norm in front cannot be combined with a residual behind");
  int NT = epi == EPI_SWIGLU ? 2 : (tiles > 0 ? tiles : 1);
  TK_REQUIRE(NT == 1 || NT == 2, "gemm_skinny: tiles=%d outside 1..2", NT);
  const int units = epi == EPI_SWIGLU ? n16 : (n16 + NT - 1) / NT;  // what one wavefront (row) owns
  bool ok;
  if (use_staged) {
    const int groups = (units + ST_WN - 1) / ST_WN;
    int WK = waves_k;
    if (WK <= 0) {
      WK = (1024 + groups * ST_WN - 1) / (groups * ST_WN);  // about a thousand wavefronts
      if (WK < 2) WK = 2;                                   // two rows a workgroup measured best
    }
    const int lds_cap = (128 * 1024) / (2 * ST_SC * MB * 1024);        // two buffers within 128 KB
    if (WK > lds_cap) WK = lds_cap;
    if (WK > K32 / ST_SC) WK = K32 / ST_SC;                            // at least a round each
    if (WK > 16 / ST_WN) WK = 16 / ST_WN;
    if (WK < 1) WK = 1;
    switch (MB) {
      case 1: ok = launch_mb<1, true>(a, epi, norm, NT, groups, WK, stream); break;
      case 2: ok = launch_mb<2, true>(a, epi, norm, NT, groups, WK, stream); break;
      case 4: ok = launch_mb<4, true>(a, epi, norm, NT, groups, WK, stream); break;
      default: ok = launch_mb<8, true>(a, epi, norm, NT, groups, WK, stream); break;
    }
  } else {
    // fewer tiles than compute units: tiles of 8 rows make twice the workgroups
    a.TH = tile_rows > 0 ? tile_rows : ((MB == 1 && units < 256) ? 8 : 16);
    const int groups = a.TH == 16 ? units : (epi == EPI_SWIGLU ? (N + 7) / 8 : ((N + 7) / 8 + NT - 1) / NT);
    int WK = waves_k;
    if (WK <= 0) {
      // a wavefront issues the loads of U steps together: best when that is all it has to do,
      // so that the whole matrix is asked for at once and the hardware queues the workgroups
      const int U = (NT + MB <= 3) ? 8 : ((NT + MB <= 6) ? 4 : 2);
      WK = K32 / (U * NT);
    }
    const int lds_cap = 65536 / (NT * MB * 64 * (int)sizeof(f32x4_t));
    if (WK > lds_cap) WK = lds_cap;
    if (WK > SK_MAX_WAVES) WK = SK_MAX_WAVES;
    if (WK > K32) WK = K32;
    if (WK < 1) WK = 1;
    switch (MB) {
      case 1: ok = launch_mb<1, false>(a, epi, norm, NT, groups, WK, stream); break;
      case 2: ok = launch_mb<2, false>(a, epi, norm, NT, groups, WK, stream); break;
      case 4: ok = launch_mb<4, false>(a, epi, norm, NT, groups, WK, stream); break;
      default: ok = launch_mb<8, false>(a, epi, norm, NT, groups, WK, stream); break;
    }
  }
  TK_REQUIRE(ok, "gemm_skinny: the kernel's local memory could not be reserved");
  TK_CHECK_LAUNCH("gemm_skinny");
  return 0;
}
