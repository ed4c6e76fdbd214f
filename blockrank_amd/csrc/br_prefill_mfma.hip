// bf16 instances of the block-sparse prefill kernel (the templates live in br_prefill_mfma_impl.h).
#include "br_prefill_mfma_impl.h"
#include <cstdlib>

namespace {

template <int D, int NW>
void launch(const BrPrefillParams& p, int grid, hipStream_t stream) {
    hipLaunchKernelGGL((br_prefill_mfma_kernel<D, NW, false>), dim3(grid), dim3(NW * 64), 0, stream, p);
}

template <int D>
int launch_resident(const BrPrefillParams& p, int n_cu, hipStream_t stream) {
    static bool armed[64] = {};    // per device: the attribute belongs to the function as loaded on that device
    const void* fn = reinterpret_cast<const void*>(&br_prefill_resident_kernel<D>);
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return -1;
    if (dev < 0 || dev >= 64 || !armed[dev]) {
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, Resident<D>::kLdsBytes) != hipSuccess) return -1;
        if (dev >= 0 && dev < 64) armed[dev] = true;
    }
    hipLaunchKernelGGL((br_prefill_resident_kernel<D>), dim3(n_cu), dim3(512), Resident<D>::kLdsBytes, stream, p);
    return 0;
}

// In view 1 the resident kernel (fused sequences) and the streaming kernel (the other sequences) run side
// by side: the resident kernel on the caller's stream, the streaming kernel on a stream of this
// library (default priority) that is forked from and joined to the caller's stream with events.
struct SideStream {
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    int device = -1;
    bool ok = false;
};
SideStream* side_stream() {
    static thread_local SideStream ss;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    if (ss.ok && ss.device == dev) return &ss;
    if (ss.ok) return nullptr;       // one device per thread; another device falls back to one stream
    if (hipStreamCreateWithFlags(&ss.stream, hipStreamNonBlocking) != hipSuccess) return nullptr;
    if (hipEventCreateWithFlags(&ss.fork, hipEventDisableTiming) != hipSuccess) return nullptr;
    if (hipEventCreateWithFlags(&ss.join, hipEventDisableTiming) != hipSuccess) return nullptr;
    ss.device = dev;
    ss.ok = true;
    return &ss;
}

}  // namespace

// Returns 0 on success, -1 if (D, NW) has no instantiation.
int br_launch_prefill_bf16(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                           hipEvent_t ev_start, hipEvent_t ev_stop) {
    const int per_cu = NW <= 4 ? 2 : 1;
    const int grid = n_cu * per_cu;
    if (ev_start) (void)hipEventRecord(ev_start, stream);
    SideStream* ss = (p.queue_view == 1 && getenv("BLOCKRANK_AMD_SIDE_STREAM") && atoi(getenv("BLOCKRANK_AMD_SIDE_STREAM")) != 0) ? side_stream() : nullptr;
    hipStream_t st_stream = stream;        // the streaming kernel's stream
    if (p.queue_view == 1) {
        if (ss) {   // fork first: the side stream waits for what precedes this call, not for the resident kernel
            if (hipEventRecord(ss->fork, stream) != hipSuccess || hipStreamWaitEvent(ss->stream, ss->fork, 0) != hipSuccess) return -2;
            st_stream = ss->stream;
        }
        if ((D == 128 ? launch_resident<128>(p, n_cu, stream) : launch_resident<64>(p, n_cu, stream)) != 0) return -1;
    }
#define BR_CASE(DD, WW)                                   \
    if (D == DD && NW == WW) {                            \
        launch<DD, WW>(p, grid, st_stream);               \
        goto launched;                                    \
    }
    BR_CASE(128, 4) BR_CASE(128, 5) BR_CASE(128, 6) BR_CASE(128, 7) BR_CASE(128, 8)
    BR_CASE(64, 4) BR_CASE(64, 5) BR_CASE(64, 6) BR_CASE(64, 7) BR_CASE(64, 8)
#undef BR_CASE
    return -1;
launched:
    if (st_stream != stream) {
        if (hipEventRecord(ss->join, ss->stream) != hipSuccess || hipStreamWaitEvent(stream, ss->join, 0) != hipSuccess) return -2;
    }
    if (ev_stop) (void)hipEventRecord(ev_stop, stream);
    if (D == 128)
        hipLaunchKernelGGL((br_finish_kernel<128>), dim3(combine_grid), dim3(256), 0, stream, p, NW);
    else
        hipLaunchKernelGGL((br_finish_kernel<64>), dim3(combine_grid), dim3(256), 0, stream, p, NW);
    return 0;
}
