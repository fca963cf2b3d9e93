// Backward of the score path (placeholder entry points until the kernels land).
#include "common.hpp"
extern "C" {
size_t kge_score_bwd_workspace(const kge_tables *, const kge_batch *) { return 0; }
int kge_score_bwd(const kge_tables *, const kge_batch *, const kge_saved *, const float *, const float *,
                  const kge_grads *, void *, size_t, void *)
{
    return KGE_EUNSUPPORTED;
}
}
