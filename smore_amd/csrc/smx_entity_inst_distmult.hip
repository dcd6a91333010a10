// Entity-pass kernels for one gradient source (see smx_entity_impl.h); one translation unit per
// source so that the sources compile in parallel.
#include "smx_entity_impl.h"

namespace smx {
template int entity_dispatch<mDistmult>(hipStream_t, const EntityArgs&, int, int);
}
