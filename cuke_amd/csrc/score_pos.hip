// Positive-triple kernels: one wavefront per (h, r, t) triple, rows gathered with
// 128-bit loads straight into registers, norms / dot products reduced with a
// wave64 butterfly.  Replaces the generated FNAME_kernel of
// pycuke1/codegen/gpu.py:182-236 (16 triples x 32 lanes per block) for the
// model definitions of apps/kge/kge.py:273-390.
#include "inspector_mid.hpp"
#include "score_pos_body.hpp"

namespace kge {

template <int MODEL, int P, int V>
__global__ __launch_bounds__(kPosWaves *kWave) void score_pos_kernel(PosArgs a, FusedInsp fi)
{
    extern __shared__ float lds[];  // TransR / RESCAL: kPosWaves * d floats; else inspector workgroups only
    if (fused_insp_block(fi, reinterpret_cast<uint32_t *>(lds))) return;
    score_pos_body<MODEL, P, V>(a, lds, (int64_t)((int)blockIdx.x - fi.blocks));
}

template <int MODEL, int P>
static int launch_pos_v(const PosArgs &a, bool vec4, const FusedInsp &fi, hipStream_t st)
{
    static_assert(kPosWaves * kWave == kMidThreads, "inspector workgroups ride with this block size");
    const dim3 grid((unsigned)ceil_div(a.B, kPosWaves) + (unsigned)fi.blocks), block(kPosWaves * kWave);
    size_t lds = (MODEL == KGE_TRANSR || MODEL == KGE_RESCAL) ? sizeof(float) * kPosWaves * (size_t)a.d : 0;
    if (fi.blocks > 0 && (size_t)fi.lds_bytes > lds) lds = (size_t)fi.lds_bytes;
    if (vec4)
        hipLaunchKernelGGL((score_pos_kernel<MODEL, P, 4>), grid, block, lds, st, a, fi);
    else
        hipLaunchKernelGGL((score_pos_kernel<MODEL, P, 1>), grid, block, lds, st, a, fi);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

// Dispatch on model / norm / vector width.  vec4 needs every row start and the
// re|im split to sit on a 16-byte boundary.
int launch_score_pos_fused(const kge_tables *tab, const kge_batch *bat, float *pos, float *resid,
                            float *side_pos, const FusedInsp *fused, hipStream_t st);

int launch_score_pos(const kge_tables *tab, const kge_batch *bat, float *pos, float *resid,
                     float *side_pos, hipStream_t st)
{
    return launch_score_pos_fused(tab, bat, pos, resid, side_pos, nullptr, st);
}

int launch_score_pos_fused(const kge_tables *tab, const kge_batch *bat, float *pos, float *resid,
                            float *side_pos, const FusedInsp *fused, hipStream_t st)
{
    if (bat->batch == 0) return KGE_OK;
    const FusedInsp fi = fused ? *fused : FusedInsp{};
    PosArgs a{tab->ent, tab->rel,      tab->aux,          bat->h,     bat->r, bat->t, bat->batch,
              (int)tab->dim, (int)tab->rel_dim, tab->gamma, pos, resid, side_pos,
              (bat->neg && bat->neg_mode == KGE_NEG_HEAD) ? 1 : 0};
    const bool complex_rows = tab->model == KGE_COMPLEX || tab->model == KGE_ROTATE;
    const bool vec4 = tab->dim % (complex_rows ? 8 : 4) == 0 && aligned16(tab->ent) &&
                      (!tab->rel || aligned16(tab->rel)) && (!tab->aux || aligned16(tab->aux)) &&
                      (!resid || aligned16(resid));
    const int p = tab->norm_p;
    switch (tab->model) {
    case KGE_TRANSE:
        return p == 1 ? launch_pos_v<KGE_TRANSE, 1>(a, vec4, fi, st) : launch_pos_v<KGE_TRANSE, 2>(a, vec4, fi, st);
    case KGE_TRANSH:
        return p == 1 ? launch_pos_v<KGE_TRANSH, 1>(a, vec4, fi, st) : launch_pos_v<KGE_TRANSH, 2>(a, vec4, fi, st);
    case KGE_TRANSR:
        if ((size_t)tab->dim * kPosWaves * sizeof(float) > 64 * 1024) return KGE_EUNSUPPORTED;
        return p == 1 ? launch_pos_v<KGE_TRANSR, 1>(a, vec4, fi, st) : launch_pos_v<KGE_TRANSR, 2>(a, vec4, fi, st);
    case KGE_RESCAL:
        if ((size_t)tab->dim * kPosWaves * sizeof(float) > 64 * 1024) return KGE_EUNSUPPORTED;
        return launch_pos_v<KGE_RESCAL, 2>(a, vec4, fi, st);
    case KGE_DISTMULT: return launch_pos_v<KGE_DISTMULT, 2>(a, vec4, fi, st);
    case KGE_COMPLEX: return launch_pos_v<KGE_COMPLEX, 2>(a, vec4, fi, st);
    case KGE_ROTATE: return launch_pos_v<KGE_ROTATE, 2>(a, vec4, fi, st);
    case KGE_TRANSF: return launch_pos_v<KGE_TRANSF, 2>(a, vec4, fi, st);
    default: return KGE_EINVAL;
    }
}

}  // namespace kge
