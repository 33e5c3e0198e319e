// Attention through low-rank latents.  A token keeps one row per layer: its normed
// key/value latent followed by a rotated key part that all heads share.  The heads'
// own key and value matrices are folded around the attention: a head's query is
// mapped into the latent's space (its unrotated part times the head's key matrix),
// attention runs with one shared "key/value head" whose values are the latents
// themselves, and the head's value matrix is applied to the result.
//
// latent_prepare_kernel: from the joint down-projection of a token, [q latent |
// key/value latent | rotated key part]: RMS norm of the two latents (float32, each
// with its weight), rotation of the key part (neighbouring pairs, float32 angles),
// the query latent to a buffer and the key row to its page slot.
// rotate_heads_kernel: rotation of a slice of every head of a row, from one buffer
// into another (the queries' rotated parts, into the folded queries' rows).
// latent_attention_kernel: one workgroup per (token, head) over the rows of the
// token's sequence, window and block bounds as in the other attention kernels;
// scores, softmax and sums are float32; tiles of 256 keys in a fixed order.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kLatThreads = 256;
constexpr int kMaxKeyDim = 1024;   // latent + rotated part
constexpr int kMaxPerThread = 4;   // value elements per thread: latents up to 1024

__device__ __forceinline__ void turn(float angle, float* c, float* s) {
  // angles reach thousands of radians: into [-pi, pi] in float64 before the float32 sine and cosine
  const double a = static_cast<double>(angle);
  const double turns = rint(a * 0.15915494309189535);
  const float reduced = static_cast<float>(fma(turns, -6.283185307179586, a));
  sincosf(reduced, s, c);
}

template <typename T>
__global__ void __launch_bounds__(kLatThreads)
    latent_prepare_kernel(const T* __restrict__ down, int q_rank, int kv_rank, int rot_dim,
                          const float* __restrict__ q_weight, const float* __restrict__ kv_weight, float eps,
                          const float* __restrict__ inv_freq, const int32_t* __restrict__ positions,
                          const int32_t* __restrict__ token_seq, const int32_t* __restrict__ tables,
                          int table_stride, T* __restrict__ q_latent, T* __restrict__ pool, int page_size,
                          int num_pages, int write_kv) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const T* row = down + static_cast<size_t>(t) * (q_rank + kv_rank + rot_dim);
  float sq_q = 0.f, sq_kv = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += kLatThreads) {
    const float x = to_float(row[i]);
    sq_q = fmaf(x, x, sq_q);
  }
  for (int i = threadIdx.x; i < kv_rank; i += kLatThreads) {
    const float x = to_float(row[q_rank + i]);
    sq_kv = fmaf(x, x, sq_kv);
  }
  const float rq = 1.f / sqrtf(block_sum(sq_q, scratch) / static_cast<float>(q_rank) + eps);
  const float rkv = 1.f / sqrtf(block_sum(sq_kv, scratch) / static_cast<float>(kv_rank) + eps);
  T* q_out = q_latent + static_cast<size_t>(t) * q_rank;
  for (int i = threadIdx.x; i < q_rank; i += kLatThreads) q_out[i] = from_float<T>(to_float(row[i]) * rq * q_weight[i]);
  if (!write_kv) return;
  const int page = tables[static_cast<size_t>(token_seq[t]) * table_stride + pos / page_size];
  if (page < 0 || page >= num_pages) return;  // a host bug; never dereferenced
  T* dst = pool + (static_cast<size_t>(page) * page_size + pos % page_size) * (kv_rank + rot_dim);
  for (int i = threadIdx.x; i < kv_rank; i += kLatThreads)
    dst[i] = from_float<T>(to_float(row[q_rank + i]) * rkv * kv_weight[i]);
  for (int i = threadIdx.x; i < rot_dim / 2; i += kLatThreads) {
    float c, s;
    turn(static_cast<float>(pos) * inv_freq[i], &c, &s);
    const float u = to_float(row[q_rank + kv_rank + 2 * i]), v = to_float(row[q_rank + kv_rank + 2 * i + 1]);
    dst[kv_rank + 2 * i] = from_float<T>(u * c - v * s);
    dst[kv_rank + 2 * i + 1] = from_float<T>(v * c + u * s);
  }
  for (int i = (rot_dim & ~1) + threadIdx.x; i < rot_dim; i += kLatThreads) dst[kv_rank + i] = row[q_rank + kv_rank + i];
}

template <typename T>
__global__ void rotate_heads_kernel(const T* __restrict__ src, int src_row, int src_head, int src_off,
                                    T* __restrict__ dst, int dst_row, int dst_head, int dst_off, int heads,
                                    int rot_dim, const float* __restrict__ inv_freq,
                                    const int32_t* __restrict__ positions) {
  const int t = blockIdx.x;
  const float pos = static_cast<float>(positions[t]);
  const int half = rot_dim / 2;
  for (int item = threadIdx.x; item < heads * half; item += blockDim.x) {
    const int h = item / half, i = item % half;
    float c, s;
    turn(pos * inv_freq[i], &c, &s);
    const T* a = src + static_cast<size_t>(t) * src_row + h * src_head + src_off + 2 * i;
    T* b = dst + static_cast<size_t>(t) * dst_row + h * dst_head + dst_off + 2 * i;
    const float u = to_float(a[0]), v = to_float(a[1]);
    b[0] = from_float<T>(u * c - v * s);
    b[1] = from_float<T>(v * c + u * s);
  }
}

template <typename T>
__global__ void __launch_bounds__(kLatThreads)
    latent_attention_kernel(const T* __restrict__ q, T* __restrict__ out, int heads, int key_dim, int v_dim,
                            const int32_t* __restrict__ positions, const int32_t* __restrict__ token_seq,
                            const int32_t* __restrict__ tables, int table_stride, const T* __restrict__ pool,
                            int page_size, int num_pages, int window, int chunk, float scale) {
  __shared__ float qs[kMaxKeyDim];
  __shared__ float probs[kLatThreads];
  __shared__ int32_t rows[kLatThreads];  // pool row of each key of the tile, -1 if masked
  __shared__ float scratch[16];
  __shared__ float partial[kLatThreads];

  const int head = blockIdx.x, t = blockIdx.y;
  const int pos = positions[t];
  const int32_t* table = tables + static_cast<size_t>(token_seq[t]) * table_stride;
  const int lo = first_key(pos, window, chunk);
  const T* qrow = q + (static_cast<size_t>(t) * heads + head) * key_dim;
  for (int d = threadIdx.x; d < key_dim; d += kLatThreads) qs[d] = to_float(qrow[d]);
  __syncthreads();

  // Sum of values: up to 256 elements, thread (g, d) sums keys g, g + groups, ... of a tile
  // for element d; beyond, every thread owns elements d, d + 256, ... for all keys of a tile.
  const bool wide = v_dim > kLatThreads;
  const int groups = wide ? 1 : kLatThreads / v_dim;
  const int g = wide ? 0 : threadIdx.x / v_dim, d0 = wide ? threadIdx.x : threadIdx.x % v_dim;
  const bool pv_active = g < groups;

  float m_run = -INFINITY, l_run = 0.f;
  float acc[kMaxPerThread] = {0.f, 0.f, 0.f, 0.f};
  for (int j0 = lo; j0 <= pos; j0 += kLatThreads) {
    const int j = j0 + threadIdx.x;
    float s = -INFINITY;
    int32_t row = -1;
    if (j <= pos) {
      const int page = table[j / page_size];
      if (page >= 0 && page < num_pages) {
        row = page * page_size + j % page_size;
        const T* kr = pool + static_cast<size_t>(row) * key_dim;
        float dot = 0.f;
        for (int e = 0; e < key_dim; ++e) dot = fmaf(qs[e], to_float(kr[e]), dot);
        s = dot * scale;
      }
    }
    const float m_new = fmaxf(m_run, block_max(s, scratch));
    const float p = (row >= 0) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m_run - m_new);  // 0 on the first tile (m_run = -inf)
    probs[threadIdx.x] = p;
    rows[threadIdx.x] = row;
    const float tile_sum = block_sum(p, scratch);  // has the barriers that publish probs/rows
    l_run = l_run * alpha + tile_sum;
    m_run = m_new;
    if (pv_active) {
      float a[kMaxPerThread] = {0.f, 0.f, 0.f, 0.f};
      const int count = (pos - j0 + 1 < kLatThreads) ? pos - j0 + 1 : kLatThreads;
      for (int jj = g; jj < count; jj += groups) {
        const int32_t r = rows[jj];
        if (r < 0) continue;
        const T* vr = pool + static_cast<size_t>(r) * key_dim;  // a key row's first v_dim elements are its values
        const float pj = probs[jj];
#pragma unroll
        for (int u = 0; u < kMaxPerThread; ++u) {
          const int d = d0 + u * kLatThreads;
          if (d < v_dim) a[u] = fmaf(pj, to_float(vr[d]), a[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < kMaxPerThread; ++u) acc[u] = acc[u] * alpha + a[u];
    }
    __syncthreads();  // probs/rows are rewritten by the next tile
  }

  T* orow = out + (static_cast<size_t>(t) * heads + head) * v_dim;
  if (wide) {
#pragma unroll
    for (int u = 0; u < kMaxPerThread; ++u) {
      const int d = d0 + u * kLatThreads;
      if (d < v_dim) orow[d] = from_float<T>(acc[u] / l_run);
    }
    return;
  }
  partial[threadIdx.x] = pv_active ? acc[0] : 0.f;
  __syncthreads();
  if (threadIdx.x < v_dim) {
    float total = 0.f;
    for (int gg = 0; gg < groups; ++gg) total += partial[gg * v_dim + threadIdx.x];
    orow[threadIdx.x] = from_float<T>(total / l_run);
  }
}

}  // namespace shk

using namespace shk;

extern "C" int shk_latent_prepare(const void* down, int dtype, int n, int q_rank, int kv_rank, int rot_dim,
                                  const float* q_weight, const float* kv_weight, float eps, const float* inv_freq,
                                  const int32_t* positions, const int32_t* token_seq, const int32_t* tables,
                                  int table_stride, void* q_latent, void* pool, int page_size, int num_pages,
                                  int write_kv, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "latent_prepare: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && q_rank > 0 && kv_rank > 0 && rot_dim >= 0 && rot_dim % 2 == 0,
              "latent_prepare: bad sizes n=%d q_rank=%d kv_rank=%d rot_dim=%d (rot_dim must be even)", n, q_rank,
              kv_rank, rot_dim);
  if (n == 0) return 0;
  SHK_REQUIRE(down && q_weight && kv_weight && positions && q_latent && (inv_freq || rot_dim == 0),
              "latent_prepare: null pointer");
  if (write_kv) {
    SHK_REQUIRE(token_seq && tables && pool, "latent_prepare: null pointer");
    SHK_REQUIRE(page_size > 0 && num_pages > 0 && table_stride > 0,
                "latent_prepare: bad cache sizes page_size=%d num_pages=%d table_stride=%d", page_size, num_pages,
                table_stride);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32)
    latent_prepare_kernel<float><<<n, kLatThreads, 0, s>>>(
        static_cast<const float*>(down), q_rank, kv_rank, rot_dim, q_weight, kv_weight, eps, inv_freq, positions,
        token_seq, tables, table_stride, static_cast<float*>(q_latent), static_cast<float*>(pool), page_size,
        num_pages, write_kv);
  else
    latent_prepare_kernel<bf16><<<n, kLatThreads, 0, s>>>(
        static_cast<const bf16*>(down), q_rank, kv_rank, rot_dim, q_weight, kv_weight, eps, inv_freq, positions,
        token_seq, tables, table_stride, static_cast<bf16*>(q_latent), static_cast<bf16*>(pool), page_size,
        num_pages, write_kv);
  SHK_LAUNCH_CHECK("latent_prepare");
  return 0;
}

extern "C" int shk_rotate_heads(const void* src, int src_row, int src_head, int src_off, void* dst, int dst_row,
                                int dst_head, int dst_off, int dtype, int n, int heads, int rot_dim,
                                const float* inv_freq, const int32_t* positions, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "rotate_heads: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && heads > 0 && rot_dim >= 0 && rot_dim % 2 == 0, "rotate_heads: bad sizes n=%d heads=%d rot_dim=%d",
              n, heads, rot_dim);
  SHK_REQUIRE(src_off >= 0 && dst_off >= 0 && src_off + rot_dim <= src_head && dst_off + rot_dim <= dst_head &&
                  heads * src_head <= src_row && heads * dst_head <= dst_row,
              "rotate_heads: the slice [%d, +%d) does not fit heads of %d (rows of %d) or [%d, +%d) heads of %d (rows of %d)",
              src_off, rot_dim, src_head, src_row, dst_off, rot_dim, dst_head, dst_row);
  if (n == 0 || rot_dim == 0) return 0;
  SHK_REQUIRE(src && dst && inv_freq && positions, "rotate_heads: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int threads = heads * rot_dim / 2 > 64 ? 256 : 64;
  if (dtype == kF32)
    rotate_heads_kernel<float><<<n, threads, 0, s>>>(static_cast<const float*>(src), src_row, src_head, src_off,
                                                     static_cast<float*>(dst), dst_row, dst_head, dst_off, heads,
                                                     rot_dim, inv_freq, positions);
  else
    rotate_heads_kernel<bf16><<<n, threads, 0, s>>>(static_cast<const bf16*>(src), src_row, src_head, src_off,
                                                    static_cast<bf16*>(dst), dst_row, dst_head, dst_off, heads,
                                                    rot_dim, inv_freq, positions);
  SHK_LAUNCH_CHECK("rotate_heads");
  return 0;
}

extern "C" int shk_latent_attention(const void* q, void* out, int dtype, int n, int heads, int key_dim, int v_dim,
                                    const int32_t* positions, const int32_t* token_seq, const int32_t* tables,
                                    int table_stride, const void* pool, int page_size, int num_pages, int window,
                                    int chunk, float scale, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "latent_attention: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && heads > 0 && heads <= 65535, "latent_attention: bad sizes n=%d heads=%d", n, heads);
  SHK_REQUIRE(key_dim > 0 && key_dim <= kMaxKeyDim && v_dim > 0 && v_dim <= key_dim &&
                  v_dim <= kMaxPerThread * kLatThreads,
              "latent_attention: rows of %d with values of %d are outside what the kernel takes (rows up to %d)",
              key_dim, v_dim, kMaxKeyDim);
  SHK_REQUIRE(page_size > 0 && num_pages > 0 && table_stride > 0,
              "latent_attention: bad cache sizes page_size=%d num_pages=%d table_stride=%d", page_size, num_pages,
              table_stride);
  SHK_REQUIRE(static_cast<int64_t>(num_pages) * page_size < (1LL << 31),
              "latent_attention: the pool has too many rows for 32-bit row indices");
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 65535, "latent_attention: at most 65535 tokens a call, got %d", n);
  SHK_REQUIRE(q && out && positions && token_seq && tables && pool, "latent_attention: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(heads, n);
  if (dtype == kF32)
    latent_attention_kernel<float><<<grid, kLatThreads, 0, s>>>(
        static_cast<const float*>(q), static_cast<float*>(out), heads, key_dim, v_dim, positions, token_seq, tables,
        table_stride, static_cast<const float*>(pool), page_size, num_pages, window, chunk, scale);
  else
    latent_attention_kernel<bf16><<<grid, kLatThreads, 0, s>>>(
        static_cast<const bf16*>(q), static_cast<bf16*>(out), heads, key_dim, v_dim, positions, token_seq, tables,
        table_stride, static_cast<const bf16*>(pool), page_size, num_pages, window, chunk, scale);
  SHK_LAUNCH_CHECK("latent_attention");
  return 0;
}
