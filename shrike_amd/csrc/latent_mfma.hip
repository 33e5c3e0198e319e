// bfloat16 attention through latents on the matrix units (gfx950).
//
// One workgroup of four wavefronts per (token, share of its keys, 64 heads); wavefront w serves 16
// query heads of the token, a lane owns one head (wavefronts without heads help to stage the rows).  All heads read the same rows (one per cached token:
// latent, then rotated key part), so a chunk of 32 rows is staged once per workgroup in LDS and
// every wavefront takes both operands from there:
//
//   S^T = R Q^T     [32 rows x 16 heads], v_mfma_f32_16x16x32_bf16 over the row's elements
//                   (padded with zeros to a multiple of 32); A = rows from LDS, 16 bytes a lane
//   softmax         running maximum and sum per head, base 2, float32; a lane holds 8 consecutive
//                   rows' scores of its head, so P^T is already in B-operand layout
//   O^T += V^T P^T  [v_dim x 16 heads]; the values are the rows' first v_dim elements, read
//                   transposed out of LDS (8 rows' element d: eight 2-byte reads; rows are
//                   padded and groups of 8 rows shifted so that these reads meet no bank twice)
//
// With nsplit > 1 the token's chunks are shared among nsplit workgroups, whose unnormalised
// results (O, maximum, sum) latent_merge_kernel joins in order (single tokens with thousands
// of rows would otherwise leave the chip idle).  Rows of up to 640 elements in multiples of 8,
// up to 128 heads; other shapes are served by latent_attention_kernel (latent.hip).
#include "api.h"
#include "common.h"

namespace shk {

typedef __bf16 lbf16x8 __attribute__((ext_vector_type(8)));
typedef float lf32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int lu32x4 __attribute__((ext_vector_type(4)));

union LFrag {
  uint4 u;
  lbf16x8 v;
  uint16_t h[8];
};

__device__ __forceinline__ float quad_lanes_max(float v) {  // over lanes j, j + 16, j + 32, j + 48
  v = fmaxf(v, __shfl_xor(v, 16, kWave));
  return fmaxf(v, __shfl_xor(v, 32, kWave));
}
__device__ __forceinline__ float quad_lanes_sum(float v) {
  v += __shfl_xor(v, 16, kWave);
  return v + __shfl_xor(v, 32, kWave);
}

constexpr int kLatentWaves = 4;  // one wavefront a SIMD: each may hold the registers of 16 heads' sums

template <int KS, int DB>  // rows of up to 32 KS elements, values of up to 16 DB
__global__ void __launch_bounds__(kLatentWaves* kWave)
    latent_attention_mfma_kernel(const bf16* __restrict__ q, bf16* __restrict__ out, int heads, int key_dim,
                                 int v_dim, const int32_t* __restrict__ positions,
                                 const int32_t* __restrict__ token_seq, const int32_t* __restrict__ tables,
                                 int table_stride, const bf16* __restrict__ pool, int page_size, int num_pages,
                                 int window, int chunk, float scale, float* __restrict__ partial, int nsplit,
                                 int n, int tpw) {
  // Rows in LDS: KS * 32 elements and 64 bytes of padding (consecutive rows start 16 banks apart: the
  // sixteen rows x four 16-byte pieces of a score operand cover the banks evenly), and every group of 8
  // rows is shifted by 32 bytes more (the four groups that a transposed value read touches at once,
  // 32 bytes each, fall into different banks).
  constexpr int STRIDE = KS * 32 + 32;
  auto at = [](int kk) { return kk * STRIDE + (kk >> 3) * 16; };
  // 16-byte pieces of a chunk that a thread stages: 32 rows of at most 4 KS pieces, 256 threads
  constexpr int kPieces = (32 * 4 * KS + kLatentWaves * kWave - 1) / (kLatentWaves * kWave);
  extern __shared__ __attribute__((aligned(16))) uint16_t rows[];  // [32][STRIDE]
  // A workgroup serves tpw tokens that follow each other in the step (1, 2 or 4; more than one only
  // where a token's heads leave wavefronts free: wavefront w then serves token w / (4 / tpw)).  (A step
  // lists a prompt's tokens in order and the last ones read the most rows: they start first, so that
  // the launch ends with light workgroups and not with its heaviest.)
  const int group = gridDim.x - 1 - blockIdx.x, z = blockIdx.y;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int wave = tid / kWave, lane = tid % kWave, j = lane % 16, g = lane / 16;
  const int wpt = kLatentWaves / tpw;  // wavefronts a token
  const int t0 = group * tpw;
  const int t_last = t0 + tpw - 1 < n - 1 ? t0 + tpw - 1 : n - 1;
  const int t = t0 + wave / wpt < n ? t0 + wave / wpt : t_last;  // (a wavefront past the step's end: idle below)
  const bool has_token = t0 + wave / wpt < n;
  const int pos = positions[t];
  const int lo = first_key(pos, window, chunk);
  const int head = (blockIdx.z * kLatentWaves + wave % wpt) * 16 + j;  // (more than 64 heads: several workgroups a token)
  const bool col_ok = has_token && head < heads;
  // Tokens of one sequence share what is staged (their rows are the same but for the newest); where a
  // workgroup's tokens belong to several sequences (single tokens of a batch, a portion's end) it
  // takes them one after the other.
  bool same = true;
  for (int i = t0 + 1; i <= t_last; ++i) same = same && token_seq[i] == token_seq[t0];
  const int passes = same ? 1 : t_last - t0 + 1;

  // the queries of this wavefront's heads as B operands: head j, elements 32 ks + 8 g ..
  LFrag qf[KS];
  const bf16* qrow = q + (static_cast<size_t>(t) * heads + (col_ok ? head : 0)) * key_dim;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    qf[ks].u = make_uint4(0, 0, 0, 0);
    const int d0 = ks * 32 + g * 8;
    if (col_ok && d0 < key_dim) qf[ks].u = *reinterpret_cast<const uint4*>(qrow + d0);
  }
  // what lies behind a row's elements stays zero for the whole kernel
  for (int i = tid; i < (32 * STRIDE + 64) / 8; i += nthreads) reinterpret_cast<uint4*>(rows)[i] = make_uint4(0, 0, 0, 0);
  __syncthreads();

  const int npieces = key_dim / 8;
  const float scale2 = scale * 1.4426950408889634f;

  float m = -INFINITY, l = 0.f;  // l: the lane's share of its head's sum until the end
  lf32x4 o[DB];                  // element 16 db + 4 g + r of the lane's head
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = lf32x4{0.f, 0.f, 0.f, 0.f};

  // A chunk's rows travel in two steps: global memory to registers (all of a thread's pieces
  // requested together, the next chunk's while this one is multiplied), registers to LDS.
  // Rows that the token does not read are zero.
  // (which row and which piece of it a thread stages does not change from chunk to chunk, and a
  // division by a number that only the launch knows costs dozens of instructions: once, up here)
  uint4 staged[kPieces];
  int piece_row[kPieces], piece_col[kPieces], piece_lds[kPieces];
#pragma unroll
  for (int u = 0; u < kPieces; ++u) {
    const int idx = tid + u * nthreads;
    piece_row[u] = idx < 32 * npieces ? idx / npieces : -1;
    piece_col[u] = (idx % npieces) * 8;
    piece_lds[u] = at(piece_row[u] < 0 ? 0 : piece_row[u]) + piece_col[u];
  }
  const int page_shift = (page_size & (page_size - 1)) == 0 ? __ffs(page_size) - 1 : -1;
  for (int pass = 0; pass < passes; ++pass) {
  // the tokens of this pass: all of the workgroup's, or its pass-th; positions rise along a portion
  const int ta = same ? t0 : t0 + pass, tb = same ? t_last : t0 + pass;
  const int stage_hi = positions[tb], stage_lo = first_key(positions[ta], window, chunk);
  const int32_t* table = tables + static_cast<size_t>(token_seq[ta]) * table_stride;
  const bool mine = has_token && t >= ta && t <= tb && head - j < heads;  // this wavefront multiplies in this pass
  const int key_begin = stage_lo & ~31;
  const int nchunks = (stage_hi - key_begin) / 32 + 1;
  const int per_split = (nchunks + nsplit - 1) / nsplit;
  const int c_first = z * per_split;
  const int c_end = c_first + per_split < nchunks ? c_first + per_split : nchunks;
  auto fetch = [&](int c) {
    const int kb = key_begin + c * 32;
#pragma unroll
    for (int u = 0; u < kPieces; ++u) {
      const int key = kb + piece_row[u];
      staged[u] = make_uint4(0, 0, 0, 0);
      if (piece_row[u] >= 0 && key >= stage_lo && key <= stage_hi) {
        const int entry = page_shift >= 0 ? key >> page_shift : key / page_size;
        const int slot = page_shift >= 0 ? key & (page_size - 1) : key % page_size;
        const int page = table[entry];
        if (page >= 0 && page < num_pages)
          staged[u] = *reinterpret_cast<const uint4*>(
              pool + (static_cast<size_t>(page) * page_size + slot) * key_dim + piece_col[u]);
      }
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int u = 0; u < kPieces; ++u)
      if (piece_row[u] >= 0) *reinterpret_cast<uint4*>(rows + piece_lds[u]) = staged[u];
  };
  if (c_first < c_end) fetch(c_first);
  for (int c = c_first; c < c_end; ++c) {
    const int kb = key_begin + c * 32;
    put();
    __syncthreads();
    if (c + 1 < c_end) fetch(c + 1);  // (the same for every thread of the workgroup)
    if (!mine) {  // a wavefront that only helps to stage in this pass
      __syncthreads();
      continue;
    }

    // ---- S^T for two tiles of 16 rows.  Row i of tile tt is row 8 (i / 4) + 4 tt + i % 4 of the
    // chunk, so that the lane's eight scores (4 tt + r) belong to the consecutive rows 8 g + e.
    lf32x4 s[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      s[tt] = lf32x4{0.f, 0.f, 0.f, 0.f};
      const int kk = 8 * (j / 4) + 4 * tt + (j % 4);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        LFrag a;
        a.u = *reinterpret_cast<const uint4*>(rows + at(kk) + ks * 32 + g * 8);
        s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[ks].v, s[tt], 0, 0, 0);
      }
    }
    float sc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = kb + 8 * g + e;
      sc[e] = (col_ok && key >= lo && key <= pos) ? s[e / 4][e % 4] * scale2 : -INFINITY;
    }
    float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
    mx = quad_lanes_max(mx);
    const float m_new = fmaxf(m, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
    float pr[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) pr[e] = __builtin_amdgcn_exp2f(sc[e] - m_safe);
    l = l * alpha + (((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7])));
    m = m_new;
    LFrag pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) pf.v[e] = static_cast<__bf16>(pr[e]);
    // ---- O^T += V^T P^T: A = element 16 db + j of rows 8 g .. 8 g + 7, B = the lane's own weights
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {  // some head's maximum rose
#pragma unroll
      for (int db = 0; db < DB; ++db) o[db] *= alpha;
    }
    const uint16_t* vrows = rows + at(8 * g) + j;  // rows 8 g .. 8 g + 7 lie STRIDE apart
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      // (packed by hand into a native vector: halves written one by one into a union's array
      // would travel through scratch memory)
      lu32x4 vw;
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2)
        vw[e2] = static_cast<uint32_t>(vrows[(2 * e2) * STRIDE + db * 16]) |
                 (static_cast<uint32_t>(vrows[(2 * e2 + 1) * STRIDE + db * 16]) << 16);
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lbf16x8, vw), pf.v, o[db], 0, 0, 0);
    }
    __syncthreads();  // the next chunk overwrites the rows
  }
  }  // passes
  l = quad_lanes_sum(l);
  if (!col_ok) return;  // (no barrier follows)

  const size_t row = static_cast<size_t>(t) * heads + head;
  if (nsplit == 1) {
    const float inv = 1.f / l;
    bf16* dst = out + row * v_dim;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int d = db * 16 + 4 * g + r;
        if (d < v_dim) dst[d] = from_float<bf16>(o[db][r] * inv);
      }
    return;
  }
  // a share's result: O [row][share][v_dim], then (maximum, sum) [row][share][2]
  const size_t all_rows = static_cast<size_t>(n) * heads;
  float* dst = partial + (row * nsplit + z) * v_dim;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int d = db * 16 + 4 * g + r;
      if (d < v_dim) dst[d] = o[db][r];
    }
  if (g == 0) {
    float* ml = partial + all_rows * nsplit * v_dim + (row * nsplit + z) * 2;
    ml[0] = m;
    ml[1] = l;
  }
}

// out[row][:] = sum_z 2^(m_z - M) O_z / sum_z 2^(m_z - M) l_z, shares in order; one wavefront a row.
__global__ void __launch_bounds__(kWave)
    latent_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out, int nsplit, int v_dim) {
  __shared__ float weight[64];
  const size_t all_rows = gridDim.x, row = blockIdx.x;
  const int lane = threadIdx.x;
  const float* ml = partial + all_rows * nsplit * v_dim + row * nsplit * 2;
  float mz = -INFINITY, lz = 0.f;
  if (lane < nsplit) mz = ml[lane * 2], lz = ml[lane * 2 + 1];
  const float mx = wave_max(mz);
  const float w = mz == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mz - mx);
  weight[lane] = w;
  __syncthreads();
  float den = 0.f;
  for (int zz = 0; zz < nsplit; ++zz) den += __shfl(w * lz, zz, kWave);
  const float inv = 1.f / den;
  const float* src = partial + row * nsplit * v_dim;
  for (int d = lane; d < v_dim; d += kWave) {
    float acc = 0.f;
    for (int zz = 0; zz < nsplit; ++zz) acc += weight[zz] * src[static_cast<size_t>(zz) * v_dim + d];
    out[row * v_dim + d] = from_float<bf16>(acc * inv);
  }
}

template <int KS, int DB>
static void launch_latent(dim3 grid, hipStream_t s, const bf16* q, bf16* out, int heads, int key_dim,
                          int v_dim, const int32_t* positions, const int32_t* token_seq, const int32_t* tables,
                          int table_stride, const bf16* pool, int page_size, int num_pages, int window, int chunk,
                          float scale, float* partial, int nsplit, int n, int tpw) {
  const size_t lds = (static_cast<size_t>(32) * (KS * 32 + 32) + 64) * sizeof(uint16_t);
  latent_attention_mfma_kernel<KS, DB><<<grid, kLatentWaves * kWave, lds, s>>>(
      q, out, heads, key_dim, v_dim, positions, token_seq, tables, table_stride, pool, page_size, num_pages, window,
      chunk, scale, partial, nsplit, n, tpw);
}

}  // namespace shk

using namespace shk;

// 1 if the matrix-instruction kernel takes the shape: rows of up to 640 elements in multiples of
// 8, values no larger than rows, up to 128 heads.
extern "C" int shk_latent_attention_supports_mfma(int heads, int key_dim, int v_dim) {
  return heads >= 1 && heads <= 128 && key_dim >= 8 && key_dim <= 640 && key_dim % 8 == 0 && v_dim >= 1 &&
         v_dim <= key_dim;
}

extern "C" int shk_latent_attention_bf16(const void* q, void* out, int n, int heads, int key_dim, int v_dim,
                                         const int32_t* positions, const int32_t* token_seq, const int32_t* tables,
                                         int table_stride, const void* pool, int page_size, int num_pages, int window,
                                         int chunk, float scale, float* partial, int nsplit, int tokens_per_group,
                                         void* stream) {
  SHK_REQUIRE(shk_latent_attention_supports_mfma(heads, key_dim, v_dim),
              "latent_attention_bf16: %d heads over rows of %d with values of %d are not served", heads, key_dim, v_dim);
  SHK_REQUIRE(n >= 0 && n <= 1 << 30 && nsplit >= 1 && nsplit <= 64 && tokens_per_group >= 1,
              "latent_attention_bf16: bad sizes n=%d nsplit=%d tokens_per_group=%d", n, nsplit, tokens_per_group);
  SHK_REQUIRE(page_size > 0 && num_pages > 0 && table_stride > 0,
              "latent_attention_bf16: bad cache sizes page_size=%d num_pages=%d table_stride=%d", page_size, num_pages,
              table_stride);
  if (n == 0) return 0;
  SHK_REQUIRE(q && out && positions && token_seq && tables && pool && (partial || nsplit == 1),
              "latent_attention_bf16: null pointer");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(pool) % 16 == 0,
              "latent_attention_bf16: q and the pool must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // tokens a workgroup: as many as its four wavefronts hold (16 heads each), if the caller allows
  int tpw = 1;
  if (tokens_per_group > 1 && heads <= 32) tpw = heads <= 16 ? 4 : 2;
  if (tpw > tokens_per_group) tpw = tokens_per_group >= 2 ? 2 : 1;
  dim3 grid((n + tpw - 1) / tpw, nsplit, (heads + 16 * kLatentWaves - 1) / (16 * kLatentWaves));
  const int ks = (key_dim + 31) / 32, db = (v_dim + 15) / 16;
#define SHK_LATENT(KS, DB)                                                                                         \
  launch_latent<KS, DB>(grid, s, static_cast<const bf16*>(q), static_cast<bf16*>(out), heads, key_dim, v_dim, \
                        positions, token_seq, tables, table_stride, static_cast<const bf16*>(pool), page_size,      \
                        num_pages, window, chunk, scale, partial, nsplit, n, tpw)
  if (ks <= 4) { if (db <= 4) SHK_LATENT(4, 4); else SHK_LATENT(4, 8); }
  else if (ks <= 8) { if (db <= 8) SHK_LATENT(8, 8); else SHK_LATENT(8, 16); }
  else if (ks <= 16) { if (db <= 16) SHK_LATENT(16, 16); else SHK_LATENT(16, 32); }
  else { if (db <= 32) SHK_LATENT(20, 32); else SHK_LATENT(20, 40); }
#undef SHK_LATENT
  if (nsplit > 1)
    latent_merge_kernel<<<static_cast<unsigned>(n) * heads, kWave, 0, s>>>(partial, static_cast<bf16*>(out), nsplit, v_dim);
  SHK_LAUNCH_CHECK("latent_attention_bf16");
  return 0;
}
