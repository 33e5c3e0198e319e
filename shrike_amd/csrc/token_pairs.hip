// Embedding lookup with a second table that is indexed by a hash of the token and
// the token before it.  The token before a step's first token of a sequence is
// state: it is kept per state slot on the device, so steps that are replayed from a
// graph or launched before the host knows their tokens find it where they look.
#include "api.h"
#include "common.h"

namespace shk {

template <typename T>
__global__ void embed_pairs_kernel(const T* __restrict__ table, const T* __restrict__ pair_table,
                                   const int32_t* __restrict__ ids,
                                   const int32_t* __restrict__ positions,
                                   const int32_t* __restrict__ token_seq,
                                   const int32_t* __restrict__ cu_q,
                                   const int32_t* __restrict__ slots, int32_t* last_token,
                                   float* __restrict__ out, int hidden, int buckets,
                                   long long mul_prev, long long mul_cur) {
  const int row = blockIdx.x;
  const int seq = token_seq[row];
  const int first = cu_q[seq];
  const int id = ids[row];
  // the token before this one: none at position 0, the row above within a step's
  // portion, else what the sequence's last step left in its slot
  int pair_row = buckets;
  if (positions[row] > 0) {
    const int prev = row > first ? ids[row - 1] : last_token[slots[seq]];
    long long h = (static_cast<long long>(prev) * mul_prev + static_cast<long long>(id) * mul_cur) % buckets;
    if (h < 0) h += buckets;
    pair_row = static_cast<int>(h);
  }
  const T* src = table + static_cast<size_t>(id) * hidden;
  const T* pair = pair_table + static_cast<size_t>(pair_row) * hidden;
  float* dst = out + static_cast<size_t>(row) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]) + to_float(pair[i]);
  if (row == first) {
    // the workgroup that read the slot is the one that writes it, after all its reads
    __syncthreads();
    if (threadIdx.x == 0) last_token[slots[seq]] = ids[cu_q[seq + 1] - 1];
  }
}

}  // namespace shk

using namespace shk;

extern "C" int shk_embed_pairs(const void* table, const void* pair_table, int dtype, const int32_t* ids,
                               const int32_t* positions, const int32_t* token_seq, const int32_t* cu_q,
                               const int32_t* slots, int32_t* last_token, float* out, int n, int hidden,
                               int vocab, int buckets, int mul_prev, int mul_cur, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "embed_pairs: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0 && vocab > 0 && buckets > 0, "embed_pairs: bad sizes n=%d hidden=%d vocab=%d buckets=%d",
              n, hidden, vocab, buckets);
  if (n == 0) return 0;
  SHK_REQUIRE(table && pair_table && ids && positions && token_seq && cu_q && slots && last_token && out,
              "embed_pairs: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int threads = hidden >= 256 ? 256 : 64;
  if (dtype == kF32)
    embed_pairs_kernel<float><<<n, threads, 0, s>>>(static_cast<const float*>(table), static_cast<const float*>(pair_table),
                                                    ids, positions, token_seq, cu_q, slots, last_token, out, hidden,
                                                    buckets, mul_prev, mul_cur);
  else
    embed_pairs_kernel<bf16><<<n, threads, 0, s>>>(static_cast<const bf16*>(table), static_cast<const bf16*>(pair_table),
                                                   ids, positions, token_seq, cu_q, slots, last_token, out, hidden,
                                                   buckets, mul_prev, mul_cur);
  SHK_LAUNCH_CHECK("embed_pairs");
  return 0;
}
