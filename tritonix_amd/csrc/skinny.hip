// Instances of the skinny (m <= 16, wavefront-level split-K) kernel and their lookup.
#include "gemm_skinny.h"
#include "registry.h"

namespace tnx {

launch_fn skinny_lookup(int dtype, int ring) {
#define TNX_SK(TAG, R) if (dtype == TAG::ID && ring == R) return &launch_skinny<TAG, R>;
  TNX_SK(TagBF16, 3) TNX_SK(TagBF16, 4) TNX_SK(TagBF16, 5) TNX_SK(TagBF16, 6)
  TNX_SK(TagF16, 3) TNX_SK(TagF16, 4) TNX_SK(TagF16, 5) TNX_SK(TagF16, 6)
#undef TNX_SK
  return nullptr;
}

}  // namespace tnx
