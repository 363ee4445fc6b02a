// The window attention of window_attention.hip on the matrix cores, bfloat16 only, for key widths
// SL_DK (a multiple of 32) and value widths SL_DV (a multiple of 16) fixed at compile time;
// SL_VK = 1: values are the first SL_DV channels of the key rows.  Same call, same meaning.
//
// What is float stays float.  The scores are products of bfloat16 numbers added up in float by
// the matrix instruction (every product is exact in float); scale, distance bias, mask, the
// running maximum and sum and the exponentials are float vector code.  A weight p is not rounded
// to bfloat16 for the second product: it is cut into three bfloat16 terms p = p1 + p2 + p3 (each
// the rounding of what the terms before left over), which carry the 24 bits of a float's
// significand, and the weighted sum of the values is three matrix instructions, one per term,
// on float accumulators.
//
// Work layout.  A column is a (token, query head) pair of one sequence and one kv head; a
// wavefront owns 16 columns, a workgroup of NW wavefronts 16 NW consecutive ones, and walks the
// blocks of 32 keys any of them sees.  A block is staged in LDS once for the workgroup: the key
// rows [32][SL_DK], and the values channel-major [SL_DV][32] (copied from the value pages, which
// are channel-major already, or scattered from the key rows).  Per block and wavefront:
//   S^T[key, column] = K[key, :] . Q[column, :]          mfma 16x16x32, A = K rows, B = Q (registers)
//   O^T[d, column] += V^T[d, key] P^T[key, column]       mfma 16x16x32, A = V^T rows, B = the terms of P
// Row i of score tile m is key 8 (i / 4) + 4 m + i % 4 of the block, so that a lane ends up with
// the weights of 8 consecutive keys of its column: the B operand of the second product as it is.
// Steps of single tokens run with NW = 1 and cut the blocks into shares over workgroups.
#include "window_attention.h"

#if defined(SL_F32)
#error "window_attention_mfma is a bfloat16 kernel; the float32 path uses window_attention.hip"
#endif
#if !defined(SL_DK) || !defined(SL_DV) || !defined(SL_VK)
#error "SL_DK, SL_DV and SL_VK must be defined"
#endif
#if SL_DK % 32 != 0 || SL_DV % 16 != 0 || SL_DK < 32 || SL_DV < 16 || SL_DV > 512 || SL_DK > 1024
#error "SL_DK must be a multiple of 32 up to 1024, SL_DV a multiple of 16 up to 512"
#endif
#if SL_VK && SL_DV > SL_DK
#error "values read from key rows cannot be wider than a key"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int DK = SL_DK, DV = SL_DV;
constexpr bool VK = SL_VK != 0;
constexpr int KK = DK / 32, DD = DV / 16;
constexpr int KROW = DK + 8;          // elements of a staged key row (the pad spreads rows over the banks)
constexpr int VROW = 40;              // elements of a staged channel row: 32 keys and a pad
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ float column_max4(float x) {      // over lanes n, n + 16, n + 32, n + 48
  x = fmaxf(x, __shfl_xor(x, 16, 64));
  return fmaxf(x, __shfl_xor(x, 32, 64));
}
__device__ __forceinline__ float column_sum4(float x) {
  x += __shfl_xor(x, 16, 64);
  return x + __shfl_xor(x, 32, 64);
}

template <int NW>
__global__ __launch_bounds__(64 * NW) void window_attention_mfma_kernel(const WindowAttention a) {
  extern __shared__ __attribute__((aligned(16))) __bf16 lds16[];
  __bf16* ks = lds16;                                  // [32][KROW]
  __bf16* vt = ks + 32 * KROW;                         // [DV][VROW]
  constexpr int THREADS = 64 * NW, COLS = 16 * NW;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 15, gq = lane >> 4;
  const int page = a.page, nkv = a.nkv;
  const int seq = blockIdx.z, kvh = blockIdx.y;
  const int g = a.nh / nkv;
  const int q0 = a.cu_q[seq], qlen = a.cu_q[seq + 1] - q0;
  const int ncols = qlen * g;
  const int tile = blockIdx.x / a.nsplit, share = blockIdx.x % a.nsplit;
  const int c0 = tile * COLS;
  if (c0 >= ncols) return;
  const int pos0 = a.positions[q0];
  const int* table = a.tables + (size_t)seq * a.max_pages;

  // the keys any column of the workgroup sees: [0, keep) and [kmin, kmax], as blocks of 32
  const int tok_first = c0 / g;
  const int c_last = c0 + COLS - 1 < ncols - 1 ? c0 + COLS - 1 : ncols - 1;
  const int kmax = pos0 + c_last / g;
  int kmin = 0;
  if (a.window > 0 && pos0 + tok_first - a.window + 1 > 0) kmin = pos0 + tok_first - a.window + 1;
  const int keep = a.keep_first < kmin ? a.keep_first : kmin;
  const int nA = keep > 0 ? (keep - 1) / 32 + 1 : 0;
  int firstB = kmin / 32;
  if (firstB < nA) firstB = nA;
  const int nB = kmax / 32 - firstB + 1 > 0 ? kmax / 32 - firstB + 1 : 0;
  const int nblk = nA + nB;
  const int i0 = (int)((long long)nblk * share / a.nsplit);
  const int i1 = (int)((long long)nblk * (share + 1) / a.nsplit);

  // this lane's column (a column past the last is computed like the last and never stored)
  int c = c0 + 16 * wave + n;
  const bool live = c < ncols;
  if (!live) c = ncols - 1;
  const int tok = c / g, head = kvh * g + c % g;
  const int pos_c = pos0 + tok;
  const int lo_c = a.window > 0 && pos_c - a.window + 1 > 0 ? pos_c - a.window + 1 : 0;
  const float scale2 = a.scale * LOG2E;
  const float slope2 = a.slopes != nullptr ? a.slopes[head] * LOG2E : 0.f;
  bf16x8 qf[KK];
  {
    const __bf16* qp = a.q + (size_t)(q0 + tok) * a.q_stride + (size_t)head * DK + 8 * gq;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const bf16x8*)(qp + 32 * kk);
  }
  f32x4 o[DD];
#pragma unroll
  for (int dd = 0; dd < DD; ++dd) o[dd] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;                        // the maximum in units of log 2
  const __bf16 zero = (__bf16)0.f;
  const bf16x8 zeros = {zero, zero, zero, zero, zero, zero, zero, zero};

  for (int i = i0; i < i1; ++i) {
    const int kbase = (i < nA ? i : firstB + (i - nA)) * 32;
    __syncthreads();                                   // the last block's readers are done
    for (int idx = tid; idx < 32 * (DK / 8); idx += THREADS) {
      const int kl = idx / (DK / 8), c8 = idx % (DK / 8), key = kbase + kl;
      bf16x8 v = zeros;
      if (key <= kmax && (key >= kmin || key < keep)) {
        const int pg = table[key / page];
        v = *(const bf16x8*)(a.kc + (((size_t)pg * nkv + kvh) * page + key % page) * DK + 8 * c8);
      }
      *(bf16x8*)(ks + kl * KROW + 8 * c8) = v;
      if (VK && 8 * c8 < DV) {
#pragma unroll
        for (int e = 0; e < 8; ++e) vt[(8 * c8 + e) * VROW + kl] = v[e];
      }
    }
    if (!VK) {
      for (int idx = tid; idx < DV * 4; idx += THREADS) {
        const int d = idx / 4, k8 = idx % 4, key0 = kbase + 8 * k8;
        bf16x8 v = zeros;
        if (key0 <= kmax && (key0 + 7 >= kmin || key0 < keep)) {
          const int pg = table[key0 / page];
          v = *(const bf16x8*)(a.vc + (((size_t)pg * nkv + kvh) * DV + d) * page + key0 % page);
#pragma unroll
          for (int e = 0; e < 8; ++e) {                // a slot of the page that holds no visible key may hold anything
            const int key = key0 + e;
            if (!(key <= kmax && (key >= kmin || key < keep))) v[e] = zero;
          }
        }
        *(bf16x8*)(vt + d * VROW + 8 * k8) = v;
      }
    }
    __syncthreads();

    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    const __bf16* kp = ks + (8 * (n / 4) + n % 4) * KROW + 8 * gq;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const bf16x8 k0 = *(const bf16x8*)(kp + 32 * kk);
      const bf16x8 k1 = *(const bf16x8*)(kp + 4 * KROW + 32 * kk);
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qf[kk], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qf[kk], s1, 0, 0, 0);
    }
    float s[8], top = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int key = kbase + 8 * gq + j;
      const bool sees = key <= pos_c && (key >= lo_c || key < a.keep_first);
      const float raw = j < 4 ? s0[j] : s1[j - 4];
      s[j] = sees ? raw * scale2 - slope2 * (float)(pos_c - key) : -INFINITY;
      top = fmaxf(top, s[j]);
    }
    const float mn = fmaxf(m, column_max4(top));
    // a column that has seen no key yet keeps m = -inf: nothing to rescale, nothing to add
    const float alpha = mn == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - mn);
    float p[8], psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      p[j] = s[j] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(s[j] - mn);
      psum += p[j];
    }
    l = l * alpha + column_sum4(psum);
    m = mn;
    bf16x8 p1, p2, p3;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      p1[j] = (__bf16)p[j];
      const float r1 = p[j] - (float)p1[j];
      p2[j] = (__bf16)r1;
      p3[j] = (__bf16)(r1 - (float)p2[j]);
    }
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) {
      const bf16x8 vf = *(const bf16x8*)(vt + (16 * dd + n) * VROW + 8 * gq);
      f32x4 acc = o[dd] * alpha;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p3, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p2, acc, 0, 0, 0);
      o[dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p1, acc, 0, 0, 0);
    }
  }
  if (!live) return;
  // this lane holds channels 16 dd + 4 gq .. + 3 of its column
  const size_t row = (size_t)(q0 + tok) * a.nh + head;
  if (a.nsplit > 1) {
    float* po = a.part_o + (row * a.nsplit + share) * DV + 4 * gq;
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) *(f32x4*)(po + 16 * dd) = o[dd];
    if (gq == 0) {
      a.part_ml[(row * a.nsplit + share) * 2] = m == -INFINITY ? m : m * (1.f / LOG2E);
      a.part_ml[(row * a.nsplit + share) * 2 + 1] = l;
    }
    return;
  }
  // every query sees itself, so m is finite here
  float top = m, extra = 0.f;
  if (a.sinks != nullptr) {
    const float sink2 = a.sinks[head] * LOG2E;
    top = fmaxf(m, sink2);
    extra = __builtin_amdgcn_exp2f(sink2 - top);
  }
  const float w = __builtin_amdgcn_exp2f(m - top);
  float f = w / (l * w + extra);
  if (a.gate != nullptr) f *= sigmoidf_(to_f(a.gate[(size_t)(q0 + tok) * a.gate_stride + head]));
  __bf16* op = a.out + row * DV + 4 * gq;
#pragma unroll
  for (int dd = 0; dd < DD; ++dd) {
    bf16x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = (__bf16)(o[dd][e] * f);
    *(bf16x4*)(op + 16 * dd) = r;
  }
}

template <int NW>
static const char* launch_mfma(const WindowAttention& a, dim3 grid, hipStream_t stream) {
  const size_t bytes = sizeof(__bf16) * ((size_t)32 * KROW + (size_t)DV * VROW);
  if (bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)window_attention_mfma_kernel<NW>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return hipGetErrorString(e);
  }
  window_attention_mfma_kernel<NW><<<grid, 64 * NW, bytes, stream>>>(a);
  return sl_launch_status();
}

extern "C" int sl_window_attention_mfma_lds_bytes() {
  return (int)(sizeof(__bf16) * ((size_t)32 * KROW + (size_t)DV * VROW));
}

// The call of sl_window_attention, for Dk == SL_DK, Dv == SL_DV and (vc == nullptr) == SL_VK.
// q rows, key rows and value rows must be 16-byte aligned.
extern "C" const char* sl_window_attention_mfma(
    const void* q, int q_stride, const void* kc, const void* vc, const int* tables, int max_pages,
    const int* cu_q, const int* positions, int num_seqs, int max_q_len, int num_tokens, int nh,
    int nkv, int Dk, int Dv, int page, float scale, int window, int keep_first, const float* slopes,
    const float* sinks, const void* gate, int gate_stride, void* out, int nsplit, float* part_o,
    float* part_ml, hipStream_t stream) {
  SL_CHECK(Dk == DK && Dv == DV && (vc == nullptr) == VK, "window attention (matrix cores): built for other widths");
  SL_CHECK(num_seqs >= 0 && max_q_len >= 1 && nh > 0 && nkv > 0 && nh % nkv == 0,
           "window attention: heads must be a positive multiple of kv heads");
  SL_CHECK(page == 16 || page == 32 || page == 64, "window attention: page size must be 16, 32 or 64");
  SL_CHECK(nkv <= 65535 && num_seqs <= 65535, "window attention: grid too large");
  SL_CHECK(window >= 0 && keep_first >= 0, "window attention: window and keep_first must be >= 0");
  SL_CHECK(nsplit >= 1 && nsplit <= 64, "window attention: 1..64 shares of the keys");
  SL_CHECK(nsplit == 1 || (part_o != nullptr && part_ml != nullptr),
           "window attention: shares of the keys need the partial buffers");
  SL_CHECK(gate == nullptr || gate_stride >= nh, "window attention: gate rows are shorter than the heads");
  SL_CHECK((uintptr_t)q % 16 == 0 && q_stride % 8 == 0 && (uintptr_t)kc % 16 == 0 && (uintptr_t)vc % 16 == 0 &&
           (uintptr_t)out % 8 == 0 && (uintptr_t)part_o % 16 == 0,
           "window attention (matrix cores): operands must be 16-byte aligned");
  if (num_seqs == 0 || num_tokens == 0) return nullptr;
  const WindowAttention a{(const act_t*)q, q_stride, (const act_t*)kc, (const act_t*)vc, tables, max_pages,
                          cu_q, positions, nh, nkv, Dk, Dv, page, scale, window, keep_first, slopes, sinks,
                          (const act_t*)gate, gate_stride, (act_t*)out, nsplit, part_o, part_ml};
  const long long cols = (long long)max_q_len * (nh / nkv);
  const int nw = cols <= 16 ? 1 : 4;
  const long long tiles = (cols + 16 * nw - 1) / (16 * nw);
  SL_CHECK(tiles * nsplit <= 1 << 30, "window attention: too many column tiles");
  const dim3 grid((unsigned)(tiles * nsplit), nkv, num_seqs);
  const char* e = nw == 1 ? launch_mfma<1>(a, grid, stream) : launch_mfma<4>(a, grid, stream);
  if (e || nsplit == 1) return e;
  window_attention_combine_kernel<<<dim3(num_tokens, nh), 64, 0, stream>>>(
      part_o, part_ml, nsplit, nh, Dv, sinks, (const act_t*)gate, gate_stride, (act_t*)out);
  return sl_launch_status();
}
