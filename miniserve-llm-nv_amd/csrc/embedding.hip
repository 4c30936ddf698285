// Token embedding: rows of the table gathered into the 32-bit residual stream.
// h[t, :] = E[token_id[t], :]   (reference: miniserve/model/qwen3.py:413,475)
#include "common.hpp"

namespace {

template <typename T>
__global__ void embedding_gather_kernel(const int32_t* __restrict__ token_ids, const T* __restrict__ table,
                                        float* __restrict__ out, int hidden, int vocab) {
  const int64_t token = blockIdx.x;
  // Ids that come from the host are checked there.  An id may also come straight from the
  // sampling kernel of the step before (a step launched before the host has read its
  // tokens), which gives -1 for a row of logits that are not finite: such a step is thrown
  // away by the host afterwards, and until then it must read inside the table.
  const int id = min(max(token_ids[token], 0), vocab - 1);
  const T* row = table + static_cast<int64_t>(id) * hidden;
  float* dst = out + token * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = ms::to_float(row[i]);
}

}  // namespace

extern "C" int ms_embedding_gather(const void* token_ids, const void* table, void* out, int num_tokens,
                                   int hidden, int vocab, int dtype, hipStream_t stream) {
  MS_REQUIRE(num_tokens > 0 && hidden > 0 && vocab > 0, "embedding_gather: empty shape");
  const int threads = hidden >= 256 ? 256 : 64;
  const dim3 grid(num_tokens);
  if (dtype == MS_F32) {
    hipLaunchKernelGGL((embedding_gather_kernel<float>), dim3(grid), dim3(threads), 0, stream, 
        static_cast<const int32_t*>(token_ids), static_cast<const float*>(table), static_cast<float*>(out), hidden, vocab);
  } else if (dtype == MS_BF16) {
    hipLaunchKernelGGL((embedding_gather_kernel<ms::bf16>), dim3(grid), dim3(threads), 0, stream, 
        static_cast<const int32_t*>(token_ids), static_cast<const ms::bf16*>(table), static_cast<float*>(out),
        hidden, vocab);
  } else {
    return ms_fail("embedding_gather: unknown dtype code %d", dtype);
  }
  MS_CHECK_LAUNCH("embedding_gather");
  return 0;
}
