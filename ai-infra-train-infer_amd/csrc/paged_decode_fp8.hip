// Instantiations of the paged decode kernel for fp8 caches (one translation unit per cache
// element type, so that the three compile side by side).
#include "paged_decode_mfma_kernel.hpp"

namespace pa {

int launch_decode_fp8(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st) {
  return launch_decode_kv<KV_FP8>(p, grid, s, st);
}

}  // namespace pa
