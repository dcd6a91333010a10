// All-entity ranking kernels for one model (see smx_rank_impl.h); one translation unit per model so
// that the models compile in parallel.
#include "smx_rank_impl.h"

namespace smx {
template int rank_dispatch<mL1>(hipStream_t, const RankArgs&, int, int, int);
}
