// Score kernels (forward, query backward) for one model (see smx_score_impl.h); one translation unit
// per model so that the models compile in parallel.
#include "smx_score_impl.h"

namespace smx {
template int score_dispatch<mDistmult>(hipStream_t, const ScoreArgs&, int, int, bool);
}
