// Shared-negative entity kernels for one model (smx_shared_impl.h); one translation unit per model so that the
// models compile in parallel.
#include "smx_shared_impl.h"

namespace smx {
template int shared_entity_dispatch<mRotate>(hipStream_t, const SharedArgs&, int, int);
}
