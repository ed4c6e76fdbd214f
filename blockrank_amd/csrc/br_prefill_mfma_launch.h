// Instances and launcher of the block-sparse prefill kernel for one 16-bit element type (the templates live in
// br_prefill_mfma_impl.h).  The including file defines BR_LAUNCH_PREFILL, the launcher's name, and, for fp16,
// BR_E16 / BR_E16_IS_F16.
#include "br_prefill_mfma_impl.h"

namespace {

// The instance is picked by what the call uses: score partials / log-sum-exp, Q rotation, or neither.
template <int D, int NW>
void launch(const BrPrefillParams& p, int grid, hipStream_t stream) {
    const bool sc = p.score_part != nullptr || p.lse != nullptr, rope = p.rope_cos != nullptr;
    if (sc && rope) hipLaunchKernelGGL((br_prefill_mfma_kernel<D, NW, false, true, true>), dim3(grid), dim3(NW * 64), 0, stream, p);
    else if (sc) hipLaunchKernelGGL((br_prefill_mfma_kernel<D, NW, false, true, false>), dim3(grid), dim3(NW * 64), 0, stream, p);
    else if (rope) hipLaunchKernelGGL((br_prefill_mfma_kernel<D, NW, false, false, true>), dim3(grid), dim3(NW * 64), 0, stream, p);
    else hipLaunchKernelGGL((br_prefill_mfma_kernel<D, NW, false, false, false>), dim3(grid), dim3(NW * 64), 0, stream, p);
}

}  // namespace

// Returns 0 on success, -1 if (D, NW) has no instantiation, 1 if the score reduction asked for with ``rank`` does not
// fit (nothing is launched in either case).
int BR_LAUNCH_PREFILL(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                           hipEvent_t ev_start, hipEvent_t ev_stop, const BrTileScoreParams* rank) {
    const int per_cu = NW <= 4 ? 2 : 1;
    const int grid = n_cu * per_cu;
    if (rank && (size_t)(rank->M - 2) * sizeof(float) > 60 * 1024) return 1;
    if (ev_start) (void)hipEventRecord(ev_start, stream);
#define BR_CASE(DD, WW)                                   \
    if (D == DD && NW == WW) {                            \
        launch<DD, WW>(p, grid, stream);                  \
        goto launched;                                    \
    }
    BR_CASE(128, 4) BR_CASE(128, 5) BR_CASE(128, 6) BR_CASE(128, 7) BR_CASE(128, 8)
    BR_CASE(64, 4) BR_CASE(64, 5) BR_CASE(64, 6) BR_CASE(64, 7) BR_CASE(64, 8)
#undef BR_CASE
    return -1;
launched:
    if (ev_stop) (void)hipEventRecord(ev_stop, stream);
    return D == 128 ? br_launch_finish<128>(p, NW, combine_grid, rank, stream) : br_launch_finish<64>(p, NW, combine_grid, rank, stream);
}
