// out[n, m] = a[n, k] @ w[m, k]^T + bias: the matrix products of the model
// (projections, feed-forward, output matrix).
//
// gemm_tiled_kernel is the general kernel: every size, float32 or bfloat16
// storage, float32 fused-multiply-add accumulation in ascending k for every
// output element.  It is the whole of the float32 path (no matrix mode of
// reduced precision is involved) and the fallback of the bfloat16 path.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kTM = 64;  // rows of a (tokens) per workgroup
constexpr int kTN = 64;  // rows of w (output features) per workgroup
constexpr int kTK = 16;  // depth of one staged slice

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
    gemm_tiled_kernel(const TI* __restrict__ a, const TI* __restrict__ w,
                      const float* __restrict__ bias, TO* __restrict__ out, int n, int m, int k,
                      int lda, int ldo, int accumulate, long long a_batch, long long w_batch,
                      long long out_batch) {
  // blockIdx.z: one of a batch of products of equal shape, operands a fixed step apart
  a += blockIdx.z * a_batch;
  w += blockIdx.z * w_batch;
  out += blockIdx.z * out_batch;
  __shared__ float as[kTK][kTM + 4];
  __shared__ float ws[kTK][kTN + 4];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int row0 = blockIdx.y * kTM, col0 = blockIdx.x * kTN;

  float acc[4][4] = {};
  for (int k0 = 0; k0 < k; k0 += kTK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = threadIdx.x + i * 256;  // 0..1023 over [64 rows][16 k]
      const int r = idx / kTK, kk = idx % kTK;
      const int gr = row0 + r, gc = col0 + r, gk = k0 + kk;
      as[kk][r] = (gr < n && gk < k) ? to_float(a[static_cast<size_t>(gr) * lda + gk]) : 0.f;
      ws[kk][r] = (gc < m && gk < k) ? to_float(w[static_cast<size_t>(gc) * k + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gr = row0 + ty * 4 + i;
    if (gr >= n) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gc = col0 + tx * 4 + j;
      if (gc >= m) continue;
      float v = acc[i][j];
      if (bias) v += bias[gc];
      TO* dst = out + static_cast<size_t>(gr) * ldo + gc;
      if (accumulate) v += to_float(*dst);
      *dst = from_float<TO>(v);
    }
  }
}

// A batch of products with few rows of a (single tokens): one wavefront per (product of the
// batch, output feature) walks that weight row once, every lane a run of it, and forms the dot
// products of up to 16 rows of a at a time; sums over the lanes in a fixed order.  Weight rows
// are read whole and once, and thousands of wavefronts keep the memory busy, where the tiled
// kernel's few workgroups would each walk a long k alone.
constexpr int kSkinnyRows = 16;

template <typename T>
__global__ void __launch_bounds__(256)
    gemm_batched_skinny_kernel(const T* __restrict__ a, const T* __restrict__ w, T* __restrict__ out, int n,
                               int m, int k, int lda, int ldo, long long a_batch, long long w_batch,
                               long long out_batch) {
  const int lane = threadIdx.x % kWave;
  const int row = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;  // output feature
  if (row >= m) return;
  const int b = blockIdx.y;
  const T* wr = w + b * w_batch + static_cast<size_t>(row) * k;
  const T* ab = a + b * a_batch;
  for (int n0 = 0; n0 < n; n0 += kSkinnyRows) {
    float acc[kSkinnyRows];
#pragma unroll
    for (int r = 0; r < kSkinnyRows; ++r) acc[r] = 0.f;
    for (int kk = lane; kk < k; kk += kWave) {
      const float wv = to_float(wr[kk]);
#pragma unroll
      for (int r = 0; r < kSkinnyRows; ++r)
        if (n0 + r < n) acc[r] = fmaf(to_float(ab[static_cast<size_t>(n0 + r) * lda + kk]), wv, acc[r]);
    }
#pragma unroll
    for (int r = 0; r < kSkinnyRows; ++r) {
      const float total = wave_sum(acc[r]);
      if (lane == 0 && n0 + r < n) out[b * out_batch + static_cast<size_t>(n0 + r) * ldo + row] = from_float<T>(total);
    }
  }
}

template <typename TI, typename TO>
static int launch_tiled(const void* a, const void* w, const float* bias, void* out, int n, int m,
                        int k, int lda, int ldo, int accumulate, hipStream_t s, int batch = 1,
                        long long a_batch = 0, long long w_batch = 0, long long out_batch = 0) {
  dim3 grid((m + kTN - 1) / kTN, (n + kTM - 1) / kTM, batch);
  gemm_tiled_kernel<TI, TO><<<grid, 256, 0, s>>>(static_cast<const TI*>(a),
                                                 static_cast<const TI*>(w), bias,
                                                 static_cast<TO*>(out), n, m, k, lda, ldo,
                                                 accumulate, a_batch, w_batch, out_batch);
  return 0;
}

}  // namespace shk

using namespace shk;

extern "C" int shk_gemm(const void* a, const void* w, const float* bias, void* out, int n, int m,
                        int k, int lda, int ldo, int in_dtype, int out_dtype, int accumulate,
                        void* stream) {
  SHK_REQUIRE(in_dtype == kF32 || in_dtype == kBF16, "gemm: unknown in_dtype %d", in_dtype);
  SHK_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "gemm: unknown out_dtype %d", out_dtype);
  SHK_REQUIRE(n >= 0 && m > 0 && k > 0, "gemm: bad sizes n=%d m=%d k=%d", n, m, k);
  SHK_REQUIRE(lda >= k && ldo >= m, "gemm: row strides lda=%d ldo=%d too small for k=%d m=%d", lda,
              ldo, k, m);
  SHK_REQUIRE(!accumulate || out_dtype == kF32, "gemm: accumulate needs a float32 output");
  SHK_REQUIRE(!(in_dtype == kF32 && out_dtype == kBF16),
              "gemm: float32 inputs with a bfloat16 output are not built");
  if (n == 0) return 0;
  SHK_REQUIRE(a && w && out, "gemm: null pointer");
  SHK_REQUIRE((n + kTM - 1) / kTM <= 65535, "gemm: too many rows (%d)", n);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_dtype == kF32)
    launch_tiled<float, float>(a, w, bias, out, n, m, k, lda, ldo, accumulate, s);
  else if (out_dtype == kF32)
    launch_tiled<bf16, float>(a, w, bias, out, n, m, k, lda, ldo, accumulate, s);
  else
    launch_tiled<bf16, bf16>(a, w, bias, out, n, m, k, lda, ldo, accumulate, s);
  SHK_LAUNCH_CHECK("gemm");
  return 0;
}

// The same batch on the matrix units for bfloat16: both operands are row-major with k innermost, which
// is the operand layout of v_mfma_f32_16x16x32_bf16 as it stands (a lane's 8 consecutive k of one row
// are one 16-byte load), so nothing passes through LDS.  A wavefront forms 16 rows x 64 features (four
// tiles that share the rows' operand); a workgroup of four wavefronts 64 x 64.  k in multiples of 8
// and 16-byte aligned rows; a wavefront's result does not depend on what else is in the step.
typedef __bf16 gbf16x8 __attribute__((ext_vector_type(8)));
typedef float gf32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256)
    gemm_batched_mfma_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w, bf16* __restrict__ out, int n,
                             int m, int k, int lda, int ldo, long long a_batch, long long w_batch,
                             long long out_batch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int i = lane % 16, kg = lane / 16;
  const int b = blockIdx.z;
  const int row = (blockIdx.y * 4 + wave) * 16 + i;  // the row of a whose operand this lane loads
  const int col0 = blockIdx.x * 64;
  const bf16* ar = a + b * a_batch + static_cast<size_t>(row < n ? row : 0) * lda + kg * 8;
  const bf16* wr[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int c = col0 + t * 16 + i;  // the feature whose weights this lane loads for tile t
    wr[t] = w + b * w_batch + static_cast<size_t>(c < m ? c : 0) * k + kg * 8;
  }
  gf32x4 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) acc[t] = gf32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k; k0 += 32) {
    const bool have = k0 + kg * 8 < k;  // (k is a multiple of 8: a piece is whole or absent)
    uint4 av = make_uint4(0, 0, 0, 0), wv[4];
    if (have && row < n) av = *reinterpret_cast<const uint4*>(ar + k0);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      wv[t] = make_uint4(0, 0, 0, 0);
      if (have && col0 + t * 16 + i < m) wv[t] = *reinterpret_cast<const uint4*>(wr[t] + k0);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(gbf16x8, wv[t]), __builtin_bit_cast(gbf16x8, av),
                                                       acc[t], 0, 0, 0);
  }
  // the products were formed transposed (features as rows): this lane holds features 4 kg + r of tile t for row i
  const int orow = (blockIdx.y * 4 + wave) * 16 + i;
  if (orow >= n) return;
  bf16* dst = out + b * out_batch + static_cast<size_t>(orow) * ldo;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int c = col0 + t * 16 + 4 * kg + r;
      if (c < m) dst[c] = from_float<bf16>(acc[t][r]);
    }
}

// A batch of products of one shape (one per head, say): product b reads a + b * a_batch
// (rows lda apart), w + b * w_batch ([m, k] contiguous) and writes out + b * out_batch.
extern "C" int shk_gemm_batched(const void* a, const void* w, void* out, int n, int m, int k, int lda,
                                int ldo, int batch, long long a_batch, long long w_batch,
                                long long out_batch, int dtype, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "gemm_batched: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && m > 0 && k > 0 && batch > 0 && batch <= 65535, "gemm_batched: bad sizes n=%d m=%d k=%d batch=%d",
              n, m, k, batch);
  SHK_REQUIRE(lda >= k && ldo >= m, "gemm_batched: row strides lda=%d ldo=%d too small for k=%d m=%d", lda, ldo, k, m);
  SHK_REQUIRE(a_batch >= 0 && w_batch >= 0 && out_batch >= m, "gemm_batched: outputs of the batch would overlap");
  if (n == 0) return 0;
  SHK_REQUIRE(a && w && out, "gemm_batched: null pointer");
  SHK_REQUIRE((n + kTM - 1) / kTM <= 65535, "gemm_batched: too many rows (%d)", n);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kBF16 && k % 8 == 0 && lda % 8 == 0 && a_batch % 8 == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(w) % 16 == 0 && (n + 63) / 64 <= 65535) {
    dim3 grid((m + 63) / 64, (n + 63) / 64, batch);
    gemm_batched_mfma_kernel<<<grid, 256, 0, s>>>(static_cast<const bf16*>(a), static_cast<const bf16*>(w),
                                                  static_cast<bf16*>(out), n, m, k, lda, ldo, a_batch, w_batch, out_batch);
  } else if (n <= 2 * kSkinnyRows && dtype == kBF16) {
    // (float32 keeps one order of summation whatever the number of rows: the tiled kernel's ascending k)
    dim3 grid((m + 3) / 4, batch);
    if (dtype == kF32)
      gemm_batched_skinny_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(a), static_cast<const float*>(w),
                                                             static_cast<float*>(out), n, m, k, lda, ldo, a_batch,
                                                             w_batch, out_batch);
    else
      gemm_batched_skinny_kernel<bf16><<<grid, 256, 0, s>>>(static_cast<const bf16*>(a), static_cast<const bf16*>(w),
                                                            static_cast<bf16*>(out), n, m, k, lda, ldo, a_batch,
                                                            w_batch, out_batch);
  } else if (dtype == kF32)
    launch_tiled<float, float>(a, w, nullptr, out, n, m, k, lda, ldo, 0, s, batch, a_batch, w_batch, out_batch);
  else
    launch_tiled<bf16, bf16>(a, w, nullptr, out, n, m, k, lda, ldo, 0, s, batch, a_batch, w_batch, out_batch);
  SHK_LAUNCH_CHECK("gemm_batched");
  return 0;
}
