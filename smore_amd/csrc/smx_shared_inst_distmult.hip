// Shared-negative entity kernels for one model (smx_shared_impl.h; this model's forward for a shared list is a
// matrix product, smx_shared_gemm.hip); one translation unit per model so that the models compile in parallel.
#include "smx_shared_impl.h"

namespace smx {
template int shared_entity_dispatch<mDistmult>(hipStream_t, const SharedArgs&, int, int);
}
