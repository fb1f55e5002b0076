// Internal interfaces between the decode-attention planner/launcher and the
// kernels. Not part of the C ABI.
#ifndef ATBMI_PA_INTERNAL_H
#define ATBMI_PA_INTERNAL_H
#include "atbmi_common.h"

namespace atbmi {

// Waves per workgroup of the scalar kernel; each wave writes its own partial.
constexpr int PA_SCALAR_WAVES = 4;
// Query heads one scalar-kernel workgroup handles.
constexpr int PA_SCALAR_HEAD_TILE = 8;

// Tokens one MFMA-kernel wave consumes per step and query heads per wave
// (the N extent of a 16x16 MFMA tile).
constexpr int PA_MFMA_STEP = 32;
constexpr int PA_MFMA_HEAD_TILE = 16;

// Scalar (VALU) kernel: any head size up to 576, any block size, any group.
// Always writes PA_SCALAR_WAVES partials per work item.
int LaunchPaScalar(const AtbmiPaShape &shape, const PaArgs &args, int numItems, hipStream_t stream);

// MFMA kernel: head sizes and block sizes listed by PaMfmaSupports.
bool PaMfmaSupports(const AtbmiPaShape &shape);
// Waves per workgroup of the instantiation that serves `shape` (8, or 4 when
// the LDS tiles of eight waves would not fit).
int PaMfmaWaves(const AtbmiPaShape &shape);
// True when the instantiation for `shape` stages one K tile per workgroup and its waves are the
// query-head tiles of one KV head (combined 576/512 cache with at least 64 query heads per KV head).
// The plan must then use one token slice and four head tiles per workgroup.
bool PaMfmaSharedTile(const AtbmiPaShape &shape);
int LaunchPaMfma(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream);

// 128-head kernel for the combined 576/512 cache (one latent KV head, any number of query heads: waves past the
// last head only stage tiles): four waves of 32 heads each share one staged latent tile. The plan must then use one
// wave range per workgroup and one head group per 128 heads or part of them. ATBMI_PA_MLA_WIDE=0 in the environment
// turns it off.
constexpr int PA_MLA_WAVES = 4;
constexpr int PA_MLA_HEADS_PER_WG = 128;
bool PaMlaWide(const AtbmiPaShape &shape);
int LaunchPaMlaWide(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream);
// Per-operand-type halves of LaunchPaMfma (one translation unit each, so the
// instantiations compile in parallel). Return -1 when the shape has no
// instantiation.
int LaunchPaMfmaF16(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream);
int LaunchPaMfmaBf16(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream);
int LaunchPaMfmaInt8(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream);

// Event brackets around the attention kernel of a call while atbmi_timing_enable is on (every n-th launch).
// TimedLaunchBegin records the first event on `stream` when this launch is one to time (launch->begin stays null
// otherwise); TimedLaunchKernelDone records the event after the attention kernel; TimedLaunchEnd records a third
// event when a merge kernel followed and queues the record for atbmi_timing_read_split.
struct TimedLaunch {
    hipEvent_t begin = nullptr;
    hipEvent_t end = nullptr;
    bool whole = false; // atbmi_timing_whole_calls: no event between the attention kernel and its merge kernel
};
int TimedLaunchBegin(hipStream_t stream, TimedLaunch *launch);
int TimedLaunchKernelDone(hipStream_t stream, const TimedLaunch &launch);
int TimedLaunchEnd(hipStream_t stream, const TimedLaunch &launch, bool merged);

// Raises a kernel's dynamic LDS limit to `ldsBytes` on the current device, once per kernel and device.
int ConfigureKernelLds(const void *kernel, int ldsBytes);

// Merges the partials of every sequence that has more than one (scalar-kernel plan).
int LaunchPaReduce(const AtbmiPaShape &shape, const PaArgs &args, int numSeqs, hipStream_t stream);
// Merges the partials the MFMA kernel left for sequences that span several wave ranges.
int LaunchPaStreamReduce(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan,
                         hipStream_t stream);

} // namespace atbmi
#endif
