// Shared-negative kernels for one model (entity side: smx_shared_impl.h, forward: smx_shared_fwd_impl.h); one
// translation unit per model so that the models compile in parallel.
#include "smx_shared_fwd_impl.h"
#include "smx_shared_impl.h"

namespace smx {
template int shared_entity_dispatch<mRotate>(hipStream_t, const SharedArgs&, int, int);
template int shared_forward_dispatch<mRotate>(hipStream_t, const SharedFwdArgs&, int);
}
