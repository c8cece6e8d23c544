// bfloat16 matrix product for few rows (decode):  C[M,N] = A[M,K] * W[N,K]^T, M <= 128,
// on the gfx950 matrix cores with 32-bit accumulation and a fused epilogue.
//
// The product is bound by reading W once.  A workgroup owns NT tiles of 16 weight
// rows and all of K; its wavefronts split K between them, each streaming its own
// part of the rows straight from memory into the operands of
// v_mfma_f32_16x16x32_bf16 (lane l holds the 8 values W[row l%16][32*step + 8*(l/16) .. +8],
// so a row is read 64 contiguous bytes at a time), and the partial sums of the
// wavefronts are added through LDS in wavefront order.  No workgroup talks to another,
// so the sum of every output has one fixed order.
//
// With the weight tile as the first operand and up to 16 tokens as the second,
//     acc[j] of lane (r = l%16, q = l/16)  =  C[token 16*mb + r][row 16*tile + 4*q + j].
//
// Epilogues: plain store, + residual, SwiGLU (the workgroup takes the same 16 rows of the
// gate and of the up projection), 32-bit store.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2, EPI_F32 = 3 };

struct SkinnyArgs {
  const bf16_t* A;
  int lda;
  const bf16_t* W;
  void* C;
  int ldc;
  const bf16_t* residual;
  int ldr;
  int M, N, K;  // N: outputs (for SwiGLU the intermediate size; W then has 2N rows, gate first)
};

__device__ __forceinline__ float silu_mul_bf16(float g, float u) {
  const float gr = round_to<bf16_t>(g), ur = round_to<bf16_t>(u);
  const float s = round_to<bf16_t>(gr / (1.0f + expf(-gr)));
  return s * ur;
}

template <int EPI>
__device__ __forceinline__ void store4(const SkinnyArgs& a, f32x4_t v, f32x4_t up, int token, int n) {
  if (token >= a.M) return;
  float o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    o[j] = v[j];
    if (EPI == EPI_SWIGLU) o[j] = silu_mul_bf16(v[j], up[j]);
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

#define SK_MAX_WAVES 16

template <int MB, int NT, int EPI>
__global__ __launch_bounds__(SK_MAX_WAVES * 64) void gemm_skinny_kernel(SkinnyArgs a) {
  extern __shared__ f32x4_t red[];  // [wave][NT*MB][64]
  constexpr int U = (NT + MB <= 2) ? 8 : ((NT + MB <= 4) ? 4 : ((NT + MB <= 8) ? 2 : 1));  // steps whose loads are in flight together
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int WK = blockDim.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int g = blockIdx.x;
  const int K32 = (a.K + 31) >> 5;
  const int ks0 = (int)((long)K32 * wave / WK), ks1 = (int)((long)K32 * (wave + 1) / WK);
  const bool k_exact = (a.K & 31) == 0;

  // rows of W this lane streams (clamped: rows past the end are masked at the store)
  const bf16_t* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int row;
    if (EPI == EPI_SWIGLU) {
      row = min(g * 16 + r, a.N - 1) + t * a.N;  // t = 0 gate, t = 1 up
    } else {
      row = min((g * NT + t) * 16 + r, a.N - 1);
    }
    wp[t] = a.W + (size_t)row * a.K + q * 8;
  }
  const bf16_t* ap[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) ap[mb] = a.A + (size_t)min(mb * 16 + r, a.M - 1) * a.lda + q * 8;

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
        for (int t = 0; t < NT; ++t) w[u][t] = *(const bf16x8_t*)(wp[t] + (size_t)(ks + u) * 32);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) av[u][mb] = *(const bf16x8_t*)(ap[mb] + (size_t)(ks + u) * 32);
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
      if (!k_ok) {
#pragma unroll
        for (int j = 0; j < 8; ++j) w[t][j] = (__bf16)0.f;
      }
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) av[mb] = *(const bf16x8_t*)(ap[mb] + off);
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[t], av[mb], acc[t][mb], 0, 0, 0);
  }

  // add the wavefronts' partial sums in wavefront order
  if (WK > 1) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) red[(wave * NT * MB + t * MB + mb) * 64 + lane] = acc[t][mb];
    __syncthreads();
  }
  constexpr int UNITS = (EPI == EPI_SWIGLU ? 1 : NT) * MB * 64;
  for (int u = tid; u < UNITS; u += blockDim.x) {
    const int l = u & 63, mb = (u >> 6) % MB, t = (u >> 6) / MB;
    const int token = mb * 16 + (l & 15), qq = l >> 4;
    f32x4_t s0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, s1 = s0;
    if (WK > 1) {
      for (int w = 0; w < WK; ++w) {
        s0 += red[(w * NT * MB + t * MB + mb) * 64 + l];
        if (EPI == EPI_SWIGLU) s1 += red[(w * NT * MB + MB + mb) * 64 + l];
      }
    } else {
      // one wavefront: unit u is this very lane's accumulator (u < 64 * NT * MB, tid == lane)
#pragma unroll
      for (int tt = 0; tt < NT; ++tt)
#pragma unroll
        for (int mm = 0; mm < MB; ++mm) {
          if (tt == t && mm == mb) s0 = acc[tt][mm];
          if (EPI == EPI_SWIGLU && tt == 1 && mm == mb) s1 = acc[tt][mm];
        }
    }
    const int n = (EPI == EPI_SWIGLU ? g : g * NT + t) * 16 + qq * 4;
    store4<EPI>(a, s0, s1, token, n);
  }
}

template <int MB, int NT>
static void launch_skinny(const SkinnyArgs& a, int epi, int groups, int WK, hipStream_t stream) {
  const dim3 grid(groups), block(WK * 64);
  const size_t lds = WK > 1 ? (size_t)WK * NT * MB * 64 * sizeof(f32x4_t) : 0;
  switch (epi) {
    case EPI_STORE:
      hipLaunchKernelGGL((gemm_skinny_kernel<MB, NT, EPI_STORE>), grid, block, lds, stream, a);
      break;
    case EPI_RESIDUAL:
      hipLaunchKernelGGL((gemm_skinny_kernel<MB, NT, EPI_RESIDUAL>), grid, block, lds, stream, a);
      break;
    case EPI_F32:
      hipLaunchKernelGGL((gemm_skinny_kernel<MB, NT, EPI_F32>), grid, block, lds, stream, a);
      break;
    default:
      break;
  }
}

template <int MB>
static void launch_skinny_swiglu(const SkinnyArgs& a, int groups, int WK, hipStream_t stream) {
  const size_t lds = WK > 1 ? (size_t)WK * 2 * MB * 64 * sizeof(f32x4_t) : 0;
  hipLaunchKernelGGL((gemm_skinny_kernel<MB, 2, EPI_SWIGLU>), dim3(groups), dim3(WK * 64), lds, stream, a);
}

// A [M, K] bfloat16 (rows lda apart), W [N, K] row-major ([2N, K] gate over up for SwiGLU),
// C [M, N].  waves_k: wavefronts that split K inside a workgroup (0 = choose);
// tiles: weight tiles of 16 rows per workgroup, 1 or 2 (0 = choose; SwiGLU always pairs gate and up).
extern "C" int tk_gemm_skinny_bf16(const void* A, int lda, const void* W, void* C, int ldc,
                                   const void* residual, int ldr, int M, int N, int K, int epi,
                                   int waves_k, int tiles, hipStream_t stream) {
  TK_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
  TK_REQUIRE(M <= 128, "gemm_skinny: at most 128 rows, got %d", M);
  TK_REQUIRE(epi >= EPI_STORE && epi <= EPI_F32, "gemm_skinny: unknown epilogue %d", epi);
  TK_REQUIRE(K % 8 == 0, "gemm_skinny: K=%d must be a multiple of 8 for the bfloat16 kernels", K);
  TK_REQUIRE(lda % 8 == 0 && ((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0,
             "gemm_skinny: rows of A and W must be 16-byte aligned (lda=%d)", lda);
  TK_REQUIRE(lda >= K && ldc >= N, "gemm_skinny: strides shorter than rows");
  TK_REQUIRE(epi != EPI_RESIDUAL || (residual && ldr >= N), "gemm_skinny: residual missing or too narrow");
  if (M == 0) return 0;
  SkinnyArgs a;
  a.A = (const bf16_t*)A; a.lda = lda; a.W = (const bf16_t*)W; a.C = C; a.ldc = ldc;
  a.residual = (const bf16_t*)residual; a.ldr = ldr; a.M = M; a.N = N; a.K = K;

  const int n16 = (N + 15) / 16;
  const int MB = M <= 16 ? 1 : (M <= 32 ? 2 : (M <= 64 ? 4 : 8));
  int NT = epi == EPI_SWIGLU ? 2 : (tiles > 0 ? tiles : (n16 >= 4096 ? 2 : 1));
  TK_REQUIRE(NT == 1 || NT == 2, "gemm_skinny: tiles=%d outside 1..2", NT);
  const int groups = epi == EPI_SWIGLU ? n16 : (n16 + NT - 1) / NT;
  const int K32 = (K + 31) / 32;
  int WK = waves_k;
  if (WK <= 0) {
    WK = (4096 + groups - 1) / groups;  // enough wavefronts in flight to cover the memory latency
    if (WK > K32 / 2) WK = K32 / 2;     // each with at least two steps
  }
  const int lds_cap = 65536 / (NT * MB * 64 * (int)sizeof(f32x4_t));
  if (WK > lds_cap) WK = lds_cap;
  if (WK > SK_MAX_WAVES) WK = SK_MAX_WAVES;
  if (WK > K32) WK = K32;
  if (WK < 1) WK = 1;
  // with one wavefront every unit of the epilogue must be a lane of it
  if (epi == EPI_SWIGLU) {
    switch (MB) {
      case 1: launch_skinny_swiglu<1>(a, groups, WK, stream); break;
      case 2: launch_skinny_swiglu<2>(a, groups, WK, stream); break;
      case 4: launch_skinny_swiglu<4>(a, groups, WK, stream); break;
      default: launch_skinny_swiglu<8>(a, groups, WK, stream); break;
    }
  } else if (NT == 1) {
    switch (MB) {
      case 1: launch_skinny<1, 1>(a, epi, groups, WK, stream); break;
      case 2: launch_skinny<2, 1>(a, epi, groups, WK, stream); break;
      case 4: launch_skinny<4, 1>(a, epi, groups, WK, stream); break;
      default: launch_skinny<8, 1>(a, epi, groups, WK, stream); break;
    }
  } else {
    switch (MB) {
      case 1: launch_skinny<1, 2>(a, epi, groups, WK, stream); break;
      case 2: launch_skinny<2, 2>(a, epi, groups, WK, stream); break;
      case 4: launch_skinny<4, 2>(a, epi, groups, WK, stream); break;
      default: launch_skinny<8, 2>(a, epi, groups, WK, stream); break;
    }
  }
  TK_CHECK_LAUNCH("gemm_skinny");
  return 0;
}

// --------------------------------------------------------------------------
// Epilogues for products that a library computed (many rows, prefill):
//   add_residual:  out = round(prod) + residual       (prod already bfloat16)
// --------------------------------------------------------------------------
template <typename T>
__global__ void add_rows_kernel(const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(to_f32<T>(x[i]) + to_f32<T>(y[i]));
}

extern "C" int tk_add(int dt, const void* x, const void* y, void* out, size_t n, hipStream_t stream) {
  if (n == 0) return 0;
  TK_REQUIRE(n < ((size_t)1 << 40), "add: too many elements");
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dt == TK_F32)
    hipLaunchKernelGGL(add_rows_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x,
                       (const float*)y, (float*)out, n);
  else
    hipLaunchKernelGGL(add_rows_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)x,
                       (const bf16_t*)y, (bf16_t*)out, n);
  TK_CHECK_LAUNCH("add");
  return 0;
}
