// Products with one small matrix per head:  y[t, h, :] = A[h] x[t, h, :]
// for all tokens t and heads h, A [heads][N][K] in the activation type, sums in
// float.  x and y are addressed by a row stride and a head stride, so the
// operands may be columns of wider buffers.  This is what a mixer needs whose
// keys and values are made per head from a shared low-rank latent: the query
// is taken to the latent's space (A[h] = Wuk[h]^T) and the attention's output
// back from it (A[h] = Wuv[h]).
//
// The general kernel: a workgroup owns 64 tokens x 64 outputs of one head; K goes
// through LDS in chunks of 16, every thread keeps 4 x 4 sums.  bfloat16 with K in
// steps of 32, N in steps of 16 and 16-byte aligned heads runs on the matrix cores:
// a wavefront owns 16 tokens x 64 outputs and reads its operands straight from
// memory, eight values a lane (rows of A are the first operand of mfma 16x16x32,
// rows of x the second), so a step of a few single tokens reads every matrix once.
#include "common.h"

constexpr int HG_TILE = 64;
constexpr int HG_CHUNK = 16;

__global__ __launch_bounds__(256) void head_products_kernel(
    const act_t* __restrict__ x, long long x_row, int x_head, const act_t* __restrict__ A,
    act_t* __restrict__ y, long long y_row, int y_head, int T, int N, int K) {
  __shared__ float xs[HG_CHUNK][HG_TILE + 1];
  __shared__ float as[HG_CHUNK][HG_TILE + 1];
  const int h = blockIdx.z, n0 = blockIdx.x * HG_TILE, t0 = blockIdx.y * HG_TILE;
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const act_t* xh = x + (size_t)h * x_head;
  const act_t* Ah = A + (size_t)h * N * K;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += HG_CHUNK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256, r = idx / HG_CHUNK, kk = idx % HG_CHUNK;
      const int k = k0 + kk;
      xs[kk][r] = (t0 + r < T && k < K) ? to_f(xh[(size_t)(t0 + r) * x_row + k]) : 0.f;
      as[kk][r] = (n0 + r < N && k < K) ? to_f(Ah[(size_t)(n0 + r) * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HG_CHUNK; ++kk) {
      float xv[4], av[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) xv[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) av[j] = as[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += xv[i] * av[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty * 4 + i;
    if (t >= T) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) y[(size_t)t * y_row + (size_t)h * y_head + n] = from_f<act_t>(acc[i][j]);
    }
  }
}

#if !defined(SL_F32)
typedef __bf16 hg_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 hg_bf16x4 __attribute__((ext_vector_type(4)));
typedef float hg_f32x4 __attribute__((ext_vector_type(4)));

// NT tiles of 16 tokens by NU tiles of 16 outputs a wavefront: 4 x 4 for many tokens (eight loads
// feed sixteen matrix instructions), 1 x 1 for a few single tokens (more wavefronts, each with a
// short chain of loads).
template <int NT, int NU>
__global__ __launch_bounds__(64) void head_products_mfma_kernel(
    const __bf16* __restrict__ x, long long x_row, int x_head, const __bf16* __restrict__ A,
    __bf16* __restrict__ y, long long y_row, int y_head, int T, int N, int K) {
  const int lane = threadIdx.x, i = lane & 15, gq = lane >> 4;
  const int h = blockIdx.z, n0 = blockIdx.x * 16 * NU, t0 = blockIdx.y * 16 * NT;
  const __bf16* xp[NT];
#pragma unroll
  for (int v = 0; v < NT; ++v) {                       // rows past the last: computed like the last, never stored
    const int t = t0 + 16 * v + i < T ? t0 + 16 * v + i : T - 1;
    xp[v] = x + (size_t)t * x_row + (size_t)h * x_head + 8 * gq;
  }
  const __bf16* ap[NU];
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int n = n0 + 16 * u + i < N ? n0 + 16 * u + i : N - 1;
    ap[u] = A + ((size_t)h * N + n) * K + 8 * gq;
  }
  hg_f32x4 acc[NT][NU];
#pragma unroll
  for (int v = 0; v < NT; ++v)
#pragma unroll
    for (int u = 0; u < NU; ++u) acc[v][u] = hg_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int k = 0; k < K; k += 32) {
    hg_bf16x8 b[NT], a[NU];
#pragma unroll
    for (int v = 0; v < NT; ++v) b[v] = *(const hg_bf16x8*)(xp[v] + k);
#pragma unroll
    for (int u = 0; u < NU; ++u) a[u] = *(const hg_bf16x8*)(ap[u] + k);
#pragma unroll
    for (int v = 0; v < NT; ++v)
#pragma unroll
      for (int u = 0; u < NU; ++u)
        acc[v][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[v], acc[v][u], 0, 0, 0);
  }
  // this lane holds outputs n0 + 16 u + 4 gq .. + 3 of tokens t0 + 16 v + i
#pragma unroll
  for (int v = 0; v < NT; ++v) {
    const int t = t0 + 16 * v + i;
    if (t >= T) continue;
    __bf16* yp = y + (size_t)t * y_row + (size_t)h * y_head + n0 + 4 * gq;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      if (n0 + 16 * u < N) {
        hg_bf16x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = (__bf16)acc[v][u][e];
        *(hg_bf16x4*)(yp + 16 * u) = r;
      }
    }
  }
}
#endif

extern "C" const char* sl_head_products(const void* x, long long x_row, int x_head, const void* A,
                                        void* y, long long y_row, int y_head, int T, int heads, int N,
                                        int K, hipStream_t stream) {
  SL_CHECK(T >= 0 && heads > 0 && N > 0 && K > 0, "head_products: sizes must be positive");
  SL_CHECK(heads <= 65535, "head_products: more than 65535 heads");
  SL_CHECK(x_head >= K && y_head >= N, "head_products: heads overlap");
  SL_CHECK(x_row >= (long long)(heads - 1) * x_head + K && y_row >= (long long)(heads - 1) * y_head + N,
           "head_products: rows are shorter than their heads");
  if (T == 0) return nullptr;
#if !defined(SL_F32)
  if (K % 32 == 0 && N % 16 == 0 && (uintptr_t)x % 16 == 0 && x_row % 8 == 0 && x_head % 8 == 0 &&
      (uintptr_t)A % 16 == 0 && (uintptr_t)y % 8 == 0 && y_row % 4 == 0 && y_head % 4 == 0 &&
      (T + 15) / 16 <= 65535) {   // (rows of A past N are clamped, their results never stored)
    if (T <= 16)
      head_products_mfma_kernel<1, 1><<<dim3(N / 16, 1, heads), 64, 0, stream>>>(
          (const __bf16*)x, x_row, x_head, (const __bf16*)A, (__bf16*)y, y_row, y_head, T, N, K);
    else if (T <= 256)
      head_products_mfma_kernel<1, 4><<<dim3((N + 63) / 64, (T + 15) / 16, heads), 64, 0, stream>>>(
          (const __bf16*)x, x_row, x_head, (const __bf16*)A, (__bf16*)y, y_row, y_head, T, N, K);
    else
      head_products_mfma_kernel<4, 4><<<dim3((N + 63) / 64, (T + 63) / 64, heads), 64, 0, stream>>>(
          (const __bf16*)x, x_row, x_head, (const __bf16*)A, (__bf16*)y, y_row, y_head, T, N, K);
    return sl_launch_status();
  }
#endif
  const dim3 grid((N + HG_TILE - 1) / HG_TILE, (T + HG_TILE - 1) / HG_TILE, heads);
  SL_CHECK(grid.y <= 65535, "head_products: too many rows");
  head_products_kernel<<<grid, 256, 0, stream>>>((const act_t*)x, x_row, x_head, (const act_t*)A,
                                                 (act_t*)y, y_row, y_head, T, N, K);
  return sl_launch_status();
}
