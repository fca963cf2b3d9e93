// TransR grouped per-relation projection (placeholder: ungrouped per-triple path).
#include "common.hpp"

namespace kge {
int launch_score_pos(const kge_tables *, const kge_batch *, float *, float *, float *, hipStream_t);
int launch_transr_fwd(const kge_tables *tab, const kge_batch *bat, float *pos, float *resid, hipStream_t st)
{
    return launch_score_pos(tab, bat, pos, resid, nullptr, st);
}
}  // namespace kge

namespace kge {
size_t transr_bwd_workspace(const kge_tables *, const kge_batch *) { return 0; }
int launch_transr_bwd(const kge_tables *, const kge_batch *, const kge_saved *, const float *,
                      const kge_grads *, void *, size_t, hipStream_t)
{
    return KGE_EUNSUPPORTED;
}
}  // namespace kge
