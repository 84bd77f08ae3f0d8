// Fast path of the fused scan + pool forward (k-mer lookup table in LDS). Placeholder: declines
// every shape so the general kernel runs.
#include "dbk_common.h"

namespace dbk_scanpool_kmer {

int fprop(hipStream_t, const float*, const float*, size_t, size_t, const uint8_t*, size_t,
          const uint32_t*, size_t, int, float*, uint32_t*)
{
    return -1;
}

}  // namespace dbk_scanpool_kmer
