// Host side of paged decode attention: shape validation, the split-KV
// planner, plan upload and kernel dispatch.
//
// The planner plays the part of the reference's PagedAttentionTiling
// (reference src/kernels/mixkernels/pagedattention/tiling/paged_attention_tiling.cpp:419-470
// and tiling/paged_attention_tiling_dependency.cpp:186-259,406-521): it decides how the
// KV range of every sequence is cut into chunks. Unlike the reference, which
// cuts by the longest sequence, chunks here are cut per sequence from its own
// length so a skewed batch still spreads evenly over the 256 CUs.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <vector>
#include "pa_internal.h"

#define ATBMI_STATIC_SCRATCH_BYTES (32ull << 20)
static __device__ __align__(256) unsigned char scratch[ATBMI_STATIC_SCRATCH_BYTES];

namespace atbmi {

namespace {
thread_local char g_lastError[512] = "";
std::mutex g_deviceMutex;
std::map<std::pair<const void *, int>, int> g_ldsConfigured; // (kernel, device) -> bytes set
std::map<int, int> g_computeUnits;                            // device -> compute units
}

int ConfigureKernelLds(const void *kernel, int ldsBytes)
{
    int dev = 0;
    ATBMI_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_deviceMutex);
    int &have = g_ldsConfigured[std::make_pair(kernel, dev)];
    if (have < ldsBytes) {
        ATBMI_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, ldsBytes));
        have = ldsBytes;
    }
    return OK;
}

int DeviceComputeUnits()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 256;
    }
    std::lock_guard<std::mutex> lock(g_deviceMutex);
    int &cus = g_computeUnits[dev];
    if (cus <= 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        cus = n;
    }
    return cus;
}

int Fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_lastError, sizeof(g_lastError), fmt, ap);
    va_end(ap);
    return code;
}

namespace {

constexpr uint64_t WS_ALIGN = 256;
constexpr int RING = 4;
constexpr int DEFAULT_CUS = 256;

uint64_t AlignUp(uint64_t v, uint64_t a)
{
    return (v + a - 1) / a * a;
}

int64_t EnvInt(const char *name, int64_t fallback)
{
    const char *v = getenv(name);
    if (!v || !*v) {
        return fallback;
    }
    char *end = nullptr;
    long long parsed = strtoll(v, &end, 10);
    return (end && *end == '\0') ? parsed : fallback;
}

struct TimingRecord {
    hipEvent_t begin;
    hipEvent_t end;    // after the attention kernel
    hipEvent_t merged; // after the merge kernel (null when the call needs none)
};
// Scratch of the entry point that allocates nothing (atbmi_pa_decode_static): the partial rows and
// log-sum-exps a plan would otherwise keep in the caller's workspace. Every device the library runs on
// holds its own copy at its own address; host code only ever uses the address hipGetSymbolAddress gave
// for the device that is current, never the array's name.
constexpr uint64_t STATIC_SCRATCH_BYTES = ATBMI_STATIC_SCRATCH_BYTES;
constexpr int MAX_DEVICES = 64;
std::mutex g_scratchMutex;
void *g_scratchPtr[MAX_DEVICES] = {};

// Address of `scratch` on the current device, looked up once per device.
int StaticScratch(void **ptr)
{
    int dev = -1;
    ATBMI_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) {
        return Fail(ERR_INVALID_PARAM, "pa_decode_static: device %d outside [0, %d)", dev, MAX_DEVICES);
    }
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    if (!g_scratchPtr[dev]) {
        void *p = nullptr;
        ATBMI_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(::scratch)));
        if (!p) {
            return Fail(ERR_RT_FAIL, "pa_decode_static: no address for the scratch array on device %d", dev);
        }
        g_scratchPtr[dev] = p;
    }
    *ptr = g_scratchPtr[dev];
    return OK;
}

std::mutex g_timingMutex;
int g_timingEvery = 0;   // 0: off; n: bracket every n-th decode launch with events
bool g_timingWhole = false; // no event between the attention kernel and its merge kernel: the call as one interval
int64_t g_timingLaunch = 0;
std::vector<TimingRecord> g_timingRecords;

} // namespace

int TimedLaunchBegin(hipStream_t stream, TimedLaunch *launch)
{
    *launch = TimedLaunch{};
    {
        std::lock_guard<std::mutex> lock(g_timingMutex);
        if (g_timingEvery <= 0 || (g_timingLaunch++ % g_timingEvery) != 0) {
            return OK;
        }
        launch->whole = g_timingWhole;
    }
    ATBMI_HIP_CHECK(hipEventCreate(&launch->begin));
    ATBMI_HIP_CHECK(hipEventCreate(&launch->end));
    ATBMI_HIP_CHECK(hipEventRecord(launch->begin, stream));
    return OK;
}

int TimedLaunchKernelDone(hipStream_t stream, const TimedLaunch &launch)
{
    if (launch.begin && !launch.whole) {
        ATBMI_HIP_CHECK(hipEventRecord(launch.end, stream));
    }
    return OK;
}

int TimedLaunchEnd(hipStream_t stream, const TimedLaunch &launch, bool merged)
{
    if (!launch.begin) {
        return OK;
    }
    TimingRecord rec{launch.begin, launch.end, nullptr};
    if (launch.whole) {
        // one interval for the whole call: its only closing event goes behind the last kernel
        (void)hipEventRecord(rec.end, stream);
    } else if (merged && hipEventCreate(&rec.merged) == hipSuccess) {
        (void)hipEventRecord(rec.merged, stream);
    }
    std::lock_guard<std::mutex> lock(g_timingMutex);
    g_timingRecords.push_back(rec);
    return OK;
}

} // namespace atbmi

using namespace atbmi;

struct AtbmiPaPlan {
    AtbmiPaShape shape;
    bool useMfma = false;
    int headTile = 1;        // query heads per workgroup (scalar kernel) or wave (MFMA kernel)
    int partialsPerItem = 1; // scalar kernel: partial slots one work item writes
    int tokenUnit = 1;       // scalar kernel: chunk lengths are multiples of this
    int mfmaWaves = 8;       // MFMA kernel: waves per workgroup
    int numCus = DEFAULT_CUS; // compute units of the device the plan was created on
    int64_t chunkOverride = 0;
    int64_t rowStartOverride = -1; // ATBMI_PA_ROW_START_STEPS (test and tuning hook): steps charged for the start of a row
    int64_t minStepsOverride = 0;

    // MFMA kernel: the stream plan (see PaStreamPlan) and its host-side pieces
    PaStreamPlan stream{};
    std::vector<PaSeq> seqTable;       // numSeqs + 1 entries
    std::vector<uint16_t> firstSeq;    // one per workgroup range
    bool streamInline = true;          // the tables fit into the kernel arguments
    bool streamNeedsReduce = false;

    std::vector<PaWorkItem> items;
    std::vector<PaSeqInfo> reduceSeqs;
    int64_t numPartials = 0;
    int32_t batch = 0;
    int64_t totalCtx = 0;
    int64_t tableEntries = 0;
    int32_t nonEmpty = 0;    // query rows: one per non-empty sequence, or one per query token of it
    int32_t maxCtx = 0;
    int64_t rowCtx = 0;      // sum over query rows of the context they attend to
    int32_t maxQueryLen = 1; // most query tokens any sequence brings
    std::vector<PaSeq> rows; // the query rows in query/output order (stepBegin unused here)
    bool causalRows = false;            // a sequence's query rows see growing prefixes of its context
    bool emptyKeepRows = false;         // a sequence without context still owns its query rows (MultiLatentAttention)
    std::vector<int32_t> causalUse;     // empty: every sequence; else one flag per sequence

    uint64_t offItems = 0, offSeqs = 0, offPartO = 0, offPartLse = 0, blobBytes = 0, wsBytes = 0;
    std::vector<uint8_t> blob; // items then reduceSeqs, as uploaded

    // Pinned staging ring for the asynchronous plan upload. A slot is reused
    // only after the copy that last read it has finished.
    void *pinned[RING] = {nullptr, nullptr, nullptr, nullptr};
    size_t pinnedCap[RING] = {0, 0, 0, 0};
    hipEvent_t copied[RING] = {nullptr, nullptr, nullptr, nullptr};
    bool inFlight[RING] = {false, false, false, false};
    int ringPos = 0;
};

extern "C" const char *atbmi_last_error(void)
{
    return g_lastError;
}

extern "C" int atbmi_device_count(void)
{
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    return n;
}

extern "C" int atbmi_pa_plan_create(const AtbmiPaShape *shape, AtbmiPaPlan **plan)
{
    if (!shape || !plan) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: null argument");
    }
    const AtbmiPaShape &s = *shape;
    if (s.qDtype != ATBMI_F16 && s.qDtype != ATBMI_BF16) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: query must be fp16 or bf16");
    }
    if (s.kvDtype != ATBMI_INT8 && s.kvDtype != s.qDtype) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: cache dtype must equal the query dtype or be int8");
    }
    if (s.numHeads <= 0 || s.numKvHeads <= 0 || s.numHeads % s.numKvHeads != 0) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: heads %d / kv heads %d", s.numHeads, s.numKvHeads);
    }
    if (s.headDimK <= 0 || s.headDimK > 576 || s.headDimV <= 0 || s.headDimV > 576) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: head sizes %d/%d outside (0,576]", s.headDimK, s.headDimV);
    }
    if (s.mlaCombined && (s.headDimV > s.headDimK || s.kvDtype == ATBMI_INT8)) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: combined cache needs Dv <= D and a 16-bit cache");
    }
    if (s.blockSize <= 0 || s.numBlocks <= 0 || s.maxBlocksPerSeq <= 0 || s.numQueryRows <= 0) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: bad block/batch extents");
    }
    if (s.hasOffset && s.kvDtype != ATBMI_INT8) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: offsets only apply to an int8 cache");
    }
    if (s.descalePacked && s.kvDtype != ATBMI_INT8) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: packed descales only apply to an int8 cache");
    }
    if (s.maskRowBy < ATBMI_PA_MASK_ROW_SEQUENCE || s.maskRowBy > ATBMI_PA_MASK_ROW_POSITION) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: maskRowBy %d", s.maskRowBy);
    }
    if (s.ropeDim != 0 && !(s.ropeDim == 64 && s.mlaCombined && s.headDimK == 576 && s.headDimV == 512 &&
                            s.kvDtype != ATBMI_INT8)) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: the split latent layout is 512 + 64 channels of a 16-bit "
                                       "combined cache, got ropeDim %d with head sizes %d / %d", s.ropeDim, s.headDimK,
                    s.headDimV);
    }
    if (s.maskSeqDiv < 0 || s.maskSeqMod < 0 || s.descaleHeads < 0) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: maskSeqDiv %d, maskSeqMod %d, descaleHeads %d", s.maskSeqDiv,
                    s.maskSeqMod, s.descaleHeads);
    }
    if ((s.descaleHeads > 0 || s.hasRazorOffset) &&
        (s.numKvHeads != 1 || s.mlaCombined || s.kvLayout != ATBMI_PA_KV_TOKEN_MAJOR)) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: descale slices by sequence and per-slot score offsets belong to "
                                       "head compression: one KV head, separate token-major caches");
    }
    if (s.descaleHeads > 0 && s.kvDtype != ATBMI_INT8) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: descaleHeads only applies to an int8 cache");
    }
    if (s.kvLayout != ATBMI_PA_KV_TOKEN_MAJOR && s.kvLayout != ATBMI_PA_KV_HEAD_MAJOR &&
        s.kvLayout != ATBMI_PA_KV_FRACTAL_NZ) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: kvLayout %d", s.kvLayout);
    }
    if (s.kvLayout == ATBMI_PA_KV_FRACTAL_NZ &&
        !(s.ropeDim == 64 && s.numKvHeads == 1 && s.blockSize >= 16 && (s.blockSize & (s.blockSize - 1)) == 0)) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: fractal-NZ caches come with the split latent layout (ropeDim 64, "
                                       "one KV head) and a power-of-two block size of at least 16");
    }
    if (s.kvLayout == ATBMI_PA_KV_HEAD_MAJOR) {
        if (s.mlaCombined) {
            return Fail(ERR_INVALID_PARAM, "pa_plan_create: a combined cache has one head; head-major blocks do not apply");
        }
        // the kernels keep a lane's offset inside one block in 32 bits
        const int64_t width = s.headDimK > s.headDimV ? s.headDimK : s.headDimV;
        if (static_cast<int64_t>(s.numKvHeads) * s.blockSize * width * 2 > 0x7fffffffLL) {
            return Fail(ERR_INVALID_PARAM, "pa_plan_create: a head-major cache block exceeds 2 GiB");
        }
    }
    if (s.hasMask && (s.maskLen <= 0 || s.maskBatchStride < 0 || s.maskHeadStride < 0)) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: mask row length %d, strides %lld / %lld", s.maskLen,
                    (long long)s.maskBatchStride, (long long)s.maskHeadStride);
    }
    AtbmiPaPlan *p = new (std::nothrow) AtbmiPaPlan();
    if (!p) {
        return Fail(ERR_OUT_OF_HOST_MEMORY, "pa_plan_create: out of host memory");
    }
    p->shape = s;
    int kernel = s.kernel;
    const char *forced = getenv("ATBMI_PA_KERNEL");
    if (kernel == ATBMI_PA_KERNEL_AUTO && forced) {
        if (!strcmp(forced, "scalar")) {
            kernel = ATBMI_PA_KERNEL_SCALAR;
        } else if (!strcmp(forced, "mfma")) {
            kernel = ATBMI_PA_KERNEL_MFMA;
        }
    }
    const bool mfmaOk = PaMfmaSupports(s);
    if (kernel == ATBMI_PA_KERNEL_MFMA && !mfmaOk) {
        delete p;
        return Fail(ERR_INVALID_PARAM, "pa_plan_create: the MFMA kernel does not cover this shape");
    }
    p->useMfma = (kernel == ATBMI_PA_KERNEL_MFMA) || (kernel == ATBMI_PA_KERNEL_AUTO && mfmaOk);
    if (p->useMfma) {
        p->headTile = PA_MFMA_HEAD_TILE;
        p->mfmaWaves = PaMfmaWaves(s);
    } else {
        p->headTile = PA_SCALAR_HEAD_TILE;
        p->partialsPerItem = PA_SCALAR_WAVES;
        p->tokenUnit = PA_SCALAR_WAVES;
    }
    p->numCus = DeviceComputeUnits();
    p->chunkOverride = EnvInt("ATBMI_PA_CHUNK_TOKENS", 0);
    p->rowStartOverride = EnvInt("ATBMI_PA_ROW_START_STEPS", -1);
    p->minStepsOverride = EnvInt("ATBMI_PA_MIN_STEPS", 0);
    *plan = p;
    return OK;
}


namespace {

// Stream plan of the MFMA kernel: every wave gets an equal share of the linear
// step space (32-token steps of all non-empty sequences, back to back).
int PlanStream(AtbmiPaPlan *plan)
{
    const AtbmiPaShape &s = plan->shape;
    const int groupSize = s.numHeads / s.numKvHeads;
    const int headTiles = (groupSize + PA_MFMA_HEAD_TILE - 1) / PA_MFMA_HEAD_TILE;
    const int virtualHeads = s.numKvHeads * headTiles;
    const int waves = plan->mfmaWaves;
    // The waves of a workgroup take different heads of one token range when the
    // head count allows it, so that the CU reads whole cache rows.
    int headsPerWg = waves;
    while (virtualHeads % headsPerWg != 0) {
        headsPerWg >>= 1;
    }
    // shared-tile instantiations: PaMfmaWaves already returned a divisor of the head-tile count
    int tokenSlices = waves / headsPerWg;
    if (PaMlaWide(s)) {
        // each wave takes two 16-head tiles: a workgroup covers 128 heads of one token range
        headsPerWg = PA_MLA_HEADS_PER_WG / PA_MFMA_HEAD_TILE;
        tokenSlices = 1;
    }
    // Several query tokens of one sequence share a pass over its context when a GQA group
    // leaves columns of the 16-wide head tile free: 16 / group tokens per pass. The 128-head kernel takes
    // them as more heads of the same pass (q and out rows of consecutive tokens follow each other in memory
    // exactly as more heads would): 128 / heads tokens.
    int fold = 1;
    if (headTiles == 1 && !PaMlaWide(s) && plan->maxQueryLen > 1 && !plan->causalRows) {
        fold = std::min(PA_MFMA_HEAD_TILE / groupSize, plan->maxQueryLen);
    }
    if (PaMlaWide(s) && plan->maxQueryLen > 1 && !plan->causalRows && s.numHeads < PA_MLA_HEADS_PER_WG) {
        fold = std::max(1, std::min(std::min(PA_MLA_HEADS_PER_WG / s.numHeads, 8), plan->maxQueryLen)); // (the kernel tells 8 tokens apart)
    }
    const int headGroups = PaMlaWide(s) ? (fold * s.numHeads + PA_MLA_HEADS_PER_WG - 1) / PA_MLA_HEADS_PER_WG
                                        : virtualHeads / headsPerWg;
    // What starting a row costs a wave, in steps (PaStreamPlan::rowStartSteps), measured on the 8B- and 70B-shaped
    // batches: a wave whose range holds the start of a row left 3 us (16-bit caches) / 8 us (int8: descales to fetch
    // and fold into the query, twice the steps per byte) later than its neighbours with the same number of steps.
    // The 128-head kernel takes whole ranges of tokens only.
    const int rowStartSteps = PaMlaWide(s) || plan->chunkOverride > 0 ? 0
                              : plan->rowStartOverride >= 0 ? static_cast<int>(plan->rowStartOverride)
                              : s.kvDtype == ATBMI_INT8 ? 3 : 1;
    try {
        plan->seqTable.clear();
        int64_t steps = 0;
        int64_t tokenSteps = 0; // the steps that hold tokens
        for (size_t r = 0; r < plan->rows.size();) {
            // consecutive rows of one sequence, `fold` at a time
            size_t e = r + 1;
            while (e < plan->rows.size() && e - r < static_cast<size_t>(fold) &&
                   plan->rows[e].tableRow == plan->rows[r].tableRow) {
                ++e;
            }
            PaSeq sq = plan->rows[r];
            sq.nTok = static_cast<int32_t>(e - r);
            sq.stepBegin = static_cast<int32_t>(steps);
            plan->seqTable.push_back(sq);
            steps += rowStartSteps + (sq.ctxLen + PA_MFMA_STEP - 1) / PA_MFMA_STEP;
            tokenSteps += (sq.ctxLen + PA_MFMA_STEP - 1) / PA_MFMA_STEP;
            r = e;
            if (steps > 0x3fffffff) {
                return Fail(ERR_INVALID_PARAM, "pa_plan_update: too many KV tokens for one call");
            }
        }
        PaSeq sentinel{};
        sentinel.stepBegin = static_cast<int32_t>(steps);
        plan->seqTable.push_back(sentinel);
        const int numSeqs = static_cast<int>(plan->seqTable.size()) - 1;

        // One workgroup per CU and head group is the most that runs at once;
        // short batches use fewer so that a wave still has a few steps to do.
        const int64_t minSteps = plan->minStepsOverride > 0 ? plan->minStepsOverride : 2;
        int64_t wgRanges = std::max<int64_t>(1, plan->numCus / headGroups);
        if (plan->chunkOverride > 0) {
            // test hook: ranges of about this many tokens
            const int64_t per = std::max<int64_t>(1, plan->chunkOverride / PA_MFMA_STEP) * tokenSlices;
            wgRanges = std::max<int64_t>(1, (steps + per - 1) / per);
        } else {
            const int64_t cap = std::max<int64_t>(1, steps / (minSteps * tokenSlices));
            wgRanges = std::min(wgRanges, cap);
        }
        if (wgRanges * tokenSlices > 0x3fffffff / 2) {
            return Fail(ERR_INVALID_PARAM, "pa_plan_update: too many ranges");
        }
        // A wave range must hold at least one step: an empty range writes no partial row, and the merge
        // kernel reads the slot of every range between a row's first and last. Surplus waves of the last
        // workgroup idle (their range index is past numWaveRanges).
        const int32_t waveRanges = static_cast<int32_t>(std::max<int64_t>(1, std::min<int64_t>(wgRanges * tokenSlices, tokenSteps)));
        wgRanges = (waveRanges + tokenSlices - 1) / tokenSlices;

        plan->firstSeq.assign(static_cast<size_t>(wgRanges), 0);
        int cursor = 0;
        for (int64_t r = 0; r < wgRanges; ++r) {
            const int32_t begin = PaRangeBegin(static_cast<int32_t>(r * tokenSlices), static_cast<int32_t>(steps),
                                               waveRanges);
            while (cursor + 1 < numSeqs && plan->seqTable[cursor + 1].stepBegin <= begin) {
                ++cursor;
            }
            plan->firstSeq[static_cast<size_t>(r)] = static_cast<uint16_t>(std::min(cursor, 0xffff));
        }
        plan->streamNeedsReduce = false;
        int32_t maxRanges = 1;
        for (int i = 0; i < numSeqs; ++i) {
            const int32_t first = PaRangeOf(plan->seqTable[i].stepBegin, static_cast<int32_t>(steps), waveRanges);
            const int32_t last = PaRangeOf(plan->seqTable[i + 1].stepBegin - 1, static_cast<int32_t>(steps), waveRanges);
            if (first != last) {
                plan->streamNeedsReduce = true;
            }
            maxRanges = std::max(maxRanges, last - first + 1);
        }

        PaStreamPlan &sp = plan->stream;
        sp = PaStreamPlan{};
        sp.numSeqs = numSeqs;
        sp.totalSteps = static_cast<int32_t>(steps);
        sp.numWaveRanges = waveRanges;
        sp.numWgRanges = static_cast<int32_t>(wgRanges);
        sp.tokenSlices = tokenSlices;
        sp.headsPerWg = headsPerWg;
        sp.headGroups = headGroups;
        sp.headTiles = headTiles;
        sp.foldTokens = fold;
        sp.maxRangesPerRow = maxRanges;
        sp.rowStartSteps = rowStartSteps;
        // firstSeq is a 16-bit table: batches beyond 65535 sequences go through memory as 16-bit too,
        // so they are refused here rather than silently truncated
        if (numSeqs > 0xffff) {
            return Fail(ERR_INVALID_PARAM, "pa_plan_update: more than 65535 non-empty sequences");
        }
        plan->streamInline = numSeqs <= PA_INLINE_SEQS && wgRanges <= PA_INLINE_RANGES;
        const uint64_t seqBytes = plan->seqTable.size() * sizeof(PaSeq);
        const uint64_t firstBytes = plan->firstSeq.size() * sizeof(uint16_t);
        if (plan->streamInline) {
            memcpy(sp.inlineSeqs, plan->seqTable.data(), seqBytes);
            memcpy(sp.inlineFirst, plan->firstSeq.data(), firstBytes);
            plan->blobBytes = 0;
            plan->blob.clear();
            plan->offItems = plan->offSeqs = 0;
        } else {
            plan->offItems = 0; // sequence table
            plan->offSeqs = AlignUp(seqBytes, 16); // first-sequence table
            plan->blobBytes = plan->offSeqs + firstBytes;
            plan->blob.assign(plan->blobBytes, 0);
            memcpy(plan->blob.data() + plan->offItems, plan->seqTable.data(), seqBytes);
            memcpy(plan->blob.data() + plan->offSeqs, plan->firstSeq.data(), firstBytes);
        }
    } catch (const std::bad_alloc &) {
        return Fail(ERR_OUT_OF_HOST_MEMORY, "pa_plan_update: out of host memory");
    }
    plan->items.clear();
    plan->reduceSeqs.clear();
    // a slot holds the partial rows of every query token of a pass
    const uint64_t slots = plan->streamNeedsReduce ? 2ull * plan->stream.numWaveRanges * fold : 0;
    plan->numPartials = static_cast<int64_t>(slots);
    plan->offPartO = AlignUp(plan->blobBytes, WS_ALIGN);
    // (partial rows of the MFMA kernels are 16-bit values of the query's type)
    const uint64_t partOBytes = slots * s.numHeads * s.headDimV * sizeof(uint16_t);
    plan->offPartLse = AlignUp(plan->offPartO + partOBytes, WS_ALIGN);
    plan->wsBytes = AlignUp(plan->offPartLse + slots * s.numHeads * sizeof(float), WS_ALIGN);
    if (plan->blobBytes == 0 && slots == 0) {
        plan->wsBytes = 0;
    }
    return OK;
}

} // namespace

extern "C" int atbmi_pa_plan_set_causal_rows(AtbmiPaPlan *plan, int32_t enable, const int32_t *perSequence,
                                             int32_t count)
{
    if (!plan || (perSequence && count <= 0)) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_set_causal_rows: null plan or %d flags", count);
    }
    try {
        plan->causalRows = enable != 0;
        plan->causalUse.clear();
        if (plan->causalRows && perSequence) {
            plan->causalUse.assign(perSequence, perSequence + count);
        }
    } catch (const std::bad_alloc &) {
        return Fail(ERR_OUT_OF_HOST_MEMORY, "pa_plan_set_causal_rows: out of host memory");
    }
    return OK;
}

extern "C" int atbmi_pa_plan_set_empty_keep_rows(AtbmiPaPlan *plan, int32_t enable)
{
    if (!plan) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_set_empty_keep_rows: null plan");
    }
    plan->emptyKeepRows = enable != 0;
    return OK;
}

extern "C" int atbmi_pa_plan_update(AtbmiPaPlan *plan, const int32_t *ctx, int32_t batch)
{
    return atbmi_pa_plan_update_multi(plan, ctx, nullptr, batch);
}

extern "C" int atbmi_pa_plan_update_multi(AtbmiPaPlan *plan, const int32_t *ctx, const int32_t *qLens, int32_t batch)
{
    if (!plan || !ctx) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_update: null argument");
    }
    const AtbmiPaShape &s = plan->shape;
    if (batch <= 0) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_update: batch %d", batch);
    }
    int64_t total = 0, tableEntries = 0, rowCtx = 0;
    int64_t nonEmpty = 0, rowsSpanned = 0;
    const int64_t maxCtx = static_cast<int64_t>(s.maxBlocksPerSeq) * s.blockSize;
    for (int32_t b = 0; b < batch; ++b) {
        if (ctx[b] < 0 || ctx[b] > maxCtx) {
            return Fail(ERR_INVALID_PARAM, "pa_plan_update: contextLens[%d]=%d outside [0,%lld]", b, ctx[b],
                        (long long)maxCtx);
        }
        if (qLens && (qLens[b] < 0 || (ctx[b] > 0 && qLens[b] > ctx[b]))) {
            return Fail(ERR_INVALID_PARAM, "pa_plan_update: queryLens[%d]=%d outside [0, contextLens = %d]", b, qLens[b],
                        ctx[b]);
        }
        if (plan->causalRows && !plan->causalUse.empty() && static_cast<int32_t>(plan->causalUse.size()) != batch) {
            return Fail(ERR_INVALID_PARAM, "pa_plan_update: causal-row flags for %d sequences, batch %d",
                        static_cast<int>(plan->causalUse.size()), batch);
        }
        if (s.hasMask && ctx[b] > s.maskLen) {
            // both kernels index a mask row by token without a bound of their own
            return Fail(ERR_INVALID_PARAM, "pa_plan_update: contextLens[%d]=%d exceeds the mask's %d tokens per row", b,
                        ctx[b], s.maskLen);
        }
        const int32_t n = ctx[b] == 0 ? 0 : (qLens ? qLens[b] : 1);
        rowsSpanned += ctx[b] == 0 && plan->emptyKeepRows ? (qLens ? qLens[b] : 1) : n;
        if (n > 0) {
            nonEmpty += n;
            total += ctx[b];
            rowCtx += static_cast<int64_t>(n) * ctx[b];
            tableEntries += (ctx[b] + s.blockSize - 1) / s.blockSize;
        }
    }
    if (rowsSpanned > s.numQueryRows) {
        return Fail(ERR_INVALID_PARAM, "pa_plan_update: %lld query rows planned but the query holds %d",
                    (long long)rowsSpanned, s.numQueryRows);
    }
    try {
        plan->rows.clear();
        int32_t nextRow = 0; // of q / out
        for (int32_t b = 0; b < batch; ++b) {
            const int32_t n = ctx[b] == 0 ? 0 : (qLens ? qLens[b] : 1);
            if (ctx[b] == 0 && plan->emptyKeepRows) {
                nextRow += qLens ? qLens[b] : 1; // rows that are never read or written
            }
            for (int32_t i = 0; i < n; ++i) {
                PaSeq row{};
                row.tableRow = b;
                row.ctxLen = ctx[b];
                if (plan->causalRows && (plan->causalUse.empty() || plan->causalUse[static_cast<size_t>(b)] != 0)) {
                    row.ctxLen = ctx[b] - n + i + 1; // (>= 1: n <= ctx[b] was checked above)
                }
                row.nTok = 1;
                const int32_t index = nextRow++;
                row.qRow = index;
                int32_t bySeq = s.maskSeqDiv > 1 ? b / s.maskSeqDiv : b;
                bySeq = s.maskSeqMod > 0 ? bySeq % s.maskSeqMod : bySeq;
                row.maskRow = s.maskRowBy == ATBMI_PA_MASK_ROW_QUERY ? index
                              : s.maskRowBy == ATBMI_PA_MASK_ROW_POSITION ? ctx[b] - n + i : bySeq;
                plan->rows.push_back(row);
            }
        }
    } catch (const std::bad_alloc &) {
        return Fail(ERR_OUT_OF_HOST_MEMORY, "pa_plan_update: out of host memory");
    }
    plan->rowCtx = rowCtx;
    plan->maxQueryLen = 1;
    for (int32_t b = 0; qLens && b < batch; ++b) {
        plan->maxQueryLen = std::max(plan->maxQueryLen, ctx[b] > 0 ? qLens[b] : 0);
    }
    plan->batch = batch;
    plan->totalCtx = total;
    plan->tableEntries = tableEntries;
    plan->nonEmpty = static_cast<int32_t>(nonEmpty);
    plan->maxCtx = *std::max_element(ctx, ctx + batch);
    plan->items.clear();
    plan->reduceSeqs.clear();

    if (plan->useMfma) {
        return PlanStream(plan);
    }

    // Chunk length: enough workgroups to load every CU several times over,
    // but chunks long enough that the per-chunk prologue/epilogue stays small.
    const int groupSize = s.numHeads / s.numKvHeads;
    const int headTiles = (groupSize + plan->headTile - 1) / plan->headTile;
    const int64_t wgPerItem = static_cast<int64_t>(s.numKvHeads) * headTiles;
    const int64_t unit = plan->tokenUnit;
    int64_t chunk = plan->chunkOverride;
    if (chunk <= 0) {
        const int64_t targetWgs = static_cast<int64_t>(plan->numCus) * 8;
        const int64_t targetItems = std::max<int64_t>(1, targetWgs / wgPerItem);
        chunk = (rowCtx + targetItems - 1) / std::max<int64_t>(1, targetItems);
        const int64_t minChunk = plan->useMfma ? 2 * unit : 64;
        chunk = std::min<int64_t>(std::max<int64_t>(chunk, minChunk), 4096);
    }
    chunk = std::max<int64_t>(unit, (chunk + unit - 1) / unit * unit);

    int64_t partials = 0;
    int32_t qRow = 0;
    try {
        for (const PaSeq &row : plan->rows) {
            const int64_t len = row.ctxLen;
            const int64_t n = (len + chunk - 1) / chunk;
            int64_t each = (len + n - 1) / n;
            each = (each + unit - 1) / unit * unit;
            const bool direct = plan->useMfma && n == 1;
            const int64_t first = partials;
            for (int64_t i = 0; i * each < len; ++i) {
                PaWorkItem it{};
                it.qRow = qRow;
                it.seq = row.tableRow;
                it.maskRow = row.maskRow;
                it.tokBegin = static_cast<int32_t>(i * each);
                it.tokEnd = static_cast<int32_t>(std::min<int64_t>(len, (i + 1) * each));
                it.direct = direct ? 1 : 0;
                it.partialBase = direct ? -1 : static_cast<int32_t>(partials);
                if (!direct) {
                    partials += plan->partialsPerItem;
                }
                plan->items.push_back(it);
            }
            if (!direct) {
                PaSeqInfo si{};
                si.qRow = qRow;
                si.firstPartial = static_cast<int32_t>(first);
                si.numPartials = static_cast<int32_t>(partials - first);
                si.ctxLen = static_cast<int32_t>(len);
                plan->reduceSeqs.push_back(si);
            }
            ++qRow;
        }
        // Longest chunks first, so the stragglers at the end of the launch are short.
        std::stable_sort(plan->items.begin(), plan->items.end(), [](const PaWorkItem &x, const PaWorkItem &y) {
            return (x.tokEnd - x.tokBegin) > (y.tokEnd - y.tokBegin);
        });
        plan->numPartials = partials;
        const uint64_t itemBytes = plan->items.size() * sizeof(PaWorkItem);
        const uint64_t seqBytes = plan->reduceSeqs.size() * sizeof(PaSeqInfo);
        plan->offItems = 0;
        plan->offSeqs = AlignUp(itemBytes, 16);
        plan->blobBytes = plan->offSeqs + seqBytes;
        plan->blob.assign(plan->blobBytes, 0);
        if (itemBytes) {
            memcpy(plan->blob.data() + plan->offItems, plan->items.data(), itemBytes);
        }
        if (seqBytes) {
            memcpy(plan->blob.data() + plan->offSeqs, plan->reduceSeqs.data(), seqBytes);
        }
    } catch (const std::bad_alloc &) {
        return Fail(ERR_OUT_OF_HOST_MEMORY, "pa_plan_update: out of host memory");
    }
    plan->offPartO = AlignUp(plan->blobBytes, WS_ALIGN);
    const uint64_t partOBytes = static_cast<uint64_t>(partials) * s.numHeads * s.headDimV * sizeof(float);
    plan->offPartLse = AlignUp(plan->offPartO + partOBytes, WS_ALIGN);
    plan->wsBytes = AlignUp(plan->offPartLse + static_cast<uint64_t>(partials) * s.numHeads * sizeof(float), WS_ALIGN);
    return OK;
}

extern "C" uint64_t atbmi_pa_plan_workspace_size(const AtbmiPaPlan *plan)
{
    return plan ? plan->wsBytes : 0;
}

extern "C" int64_t atbmi_pa_plan_num_chunks(const AtbmiPaPlan *plan)
{
    if (!plan) {
        return 0;
    }
    return plan->useMfma ? static_cast<int64_t>(plan->stream.numWaveRanges)
                         : static_cast<int64_t>(plan->items.size());
}

extern "C" uint64_t atbmi_pa_plan_algorithmic_bytes(const AtbmiPaPlan *plan)
{
    if (!plan) {
        return 0;
    }
    const AtbmiPaShape &s = plan->shape;
    const uint64_t kvSize = s.kvDtype == ATBMI_INT8 ? 1 : 2;
    const uint64_t perToken =
        static_cast<uint64_t>(s.numKvHeads) * (s.mlaCombined ? s.headDimK : s.headDimK + s.headDimV) * kvSize;
    uint64_t bytes = static_cast<uint64_t>(plan->totalCtx) * perToken;
    bytes += static_cast<uint64_t>(plan->nonEmpty) * s.numHeads * (s.headDimK + s.headDimV) * 2;
    bytes += static_cast<uint64_t>(plan->tableEntries) * 4 + static_cast<uint64_t>(plan->batch) * 4;
    if (s.kvDtype == ATBMI_INT8) {
        const uint64_t vec = static_cast<uint64_t>(s.numKvHeads) * (s.headDimK + s.headDimV) * 4;
        bytes += vec * (s.hasOffset ? 2 : 1);
    }
    if (s.hasMask) {
        // each distinct mask row once, over the tokens attended to
        const uint64_t tokens = s.maskBatchStride ? static_cast<uint64_t>(plan->rowCtx)
                                                  : static_cast<uint64_t>(plan->maxCtx);
        bytes += tokens * (s.maskHeadStride ? s.numHeads : 1) * 2;
    }
    if (s.hasLogN) {
        bytes += static_cast<uint64_t>(plan->batch) * 4;
    }
    if (s.hasRazorOffset) {
        bytes += static_cast<uint64_t>(plan->totalCtx) * 4; // one score offset per cache slot attended to
    }
    if (plan->nonEmpty > 0 && plan->rows.size() > 0 && plan->rowCtx != plan->totalCtx) {
        bytes += static_cast<uint64_t>(plan->batch) * 4; // the query lengths
    }
    return bytes;
}

extern "C" void atbmi_pa_plan_destroy(AtbmiPaPlan *plan)
{
    if (!plan) {
        return;
    }
    for (int i = 0; i < RING; ++i) {
        if (plan->copied[i]) {
            if (plan->inFlight[i]) {
                (void)hipEventSynchronize(plan->copied[i]);
            }
            (void)hipEventDestroy(plan->copied[i]);
        }
        if (plan->pinned[i]) {
            (void)hipHostFree(plan->pinned[i]);
        }
    }
    delete plan;
}

namespace {

// Copies the plan blob into the next pinned slot and enqueues its upload.
int UploadPlan(AtbmiPaPlan *plan, void *workspace, hipStream_t stream)
{
    if (plan->blobBytes == 0) {
        return OK;
    }
    const int slot = plan->ringPos;
    plan->ringPos = (plan->ringPos + 1) % RING;
    if (plan->inFlight[slot]) {
        ATBMI_HIP_CHECK(hipEventSynchronize(plan->copied[slot]));
        plan->inFlight[slot] = false;
    }
    if (plan->pinnedCap[slot] < plan->blobBytes) {
        if (plan->pinned[slot]) {
            ATBMI_HIP_CHECK(hipHostFree(plan->pinned[slot]));
            plan->pinned[slot] = nullptr;
            plan->pinnedCap[slot] = 0;
        }
        const size_t cap = static_cast<size_t>(AlignUp(plan->blobBytes * 2, 4096));
        ATBMI_HIP_CHECK(hipHostMalloc(&plan->pinned[slot], cap, hipHostMallocDefault));
        plan->pinnedCap[slot] = cap;
    }
    if (!plan->copied[slot]) {
        ATBMI_HIP_CHECK(hipEventCreateWithFlags(&plan->copied[slot], hipEventDisableTiming));
    }
    memcpy(plan->pinned[slot], plan->blob.data(), plan->blobBytes);
    ATBMI_HIP_CHECK(hipMemcpyAsync(workspace, plan->pinned[slot], plan->blobBytes, hipMemcpyHostToDevice, stream));
    ATBMI_HIP_CHECK(hipEventRecord(plan->copied[slot], stream));
    plan->inFlight[slot] = true;
    return OK;
}

} // namespace

namespace {

// Both decode entry points. `mayAllocate` false: no plan upload (its pinned staging ring is allocated on
// demand) and no timing events.
int DecodeImpl(AtbmiPaPlan *plan, const AtbmiPaTensors *t, void *workspace, uint64_t workspaceBytes,
               void *streamHandle, bool mayAllocate)
{
    const AtbmiPaShape &s = plan->shape;
    if (!t->query || !t->keyCache || !t->blockTables || !t->out || (!s.mlaCombined && !t->valueCache)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: a required tensor is null");
    }
    if (s.kvDtype == ATBMI_INT8 && (!t->kScale || !t->vScale)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: int8 cache needs kScale and vScale");
    }
    if (s.hasRazorOffset && !t->razorOffset) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: hasRazorOffset needs razorOffset");
    }
    if (s.hasOffset && (!t->kOffset || !t->vOffset)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: hasOffset needs kOffset and vOffset");
    }
    if (s.ropeDim != 0 && (!t->queryRope || !t->keyRopeCache)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: the split latent layout needs queryRope and keyRopeCache");
    }
    if (t->lse && s.kvDtype == ATBMI_INT8) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: no log-sum-exp output with an int8 cache");
    }
    if ((s.hasMask && !t->mask) || (s.hasLogN && !t->logN)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: the plan was made with a mask / logN, none given");
    }
    if (plan->wsBytes > 0 && (!workspace || workspaceBytes < plan->wsBytes)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: workspace of %llu bytes, %llu needed",
                    (unsigned long long)workspaceBytes, (unsigned long long)plan->wsBytes);
    }
    if (plan->wsBytes > 0 && reinterpret_cast<uintptr_t>(workspace) % 16 != 0) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: workspace must be 16-byte aligned");
    }
    hipStream_t stream = static_cast<hipStream_t>(streamHandle);
    int rc = mayAllocate ? UploadPlan(plan, workspace, stream) : OK;
    if (rc != OK) {
        return rc;
    }

    uint8_t *ws = static_cast<uint8_t *>(workspace);
    PaArgs a{};
    a.q = t->query;
    a.kc = t->keyCache;
    a.vc = s.mlaCombined ? t->keyCache : t->valueCache;
    a.tables = t->blockTables;
    a.kScale = t->kScale;
    a.kOff = s.hasOffset ? t->kOffset : nullptr;
    a.vScale = t->vScale;
    a.vOff = s.hasOffset ? t->vOffset : nullptr;
    a.out = t->out;
    a.items = reinterpret_cast<const PaWorkItem *>(ws + plan->offItems);
    a.seqs = reinterpret_cast<const PaSeqInfo *>(ws + plan->offSeqs);
    a.partO = reinterpret_cast<float *>(ws + plan->offPartO);
    a.partLse = reinterpret_cast<float *>(ws + plan->offPartLse);
    a.H = s.numHeads;
    a.G = s.numKvHeads;
    a.D = s.headDimK;
    a.Dv = s.headDimV;
    a.blockSize = s.blockSize;
    a.maxBlocksPerSeq = s.maxBlocksPerSeq;
    a.qIsBf16 = s.qDtype == ATBMI_BF16;
    a.groupSize = s.numHeads / s.numKvHeads;
    a.qkScale = s.qkScale;
    a.qScale = (s.qScale == 0.0f || s.qScale == 1.0f) ? 0.0f : s.qScale;
    if (s.kvLayout == ATBMI_PA_KV_HEAD_MAJOR) {
        a.blockRows = s.blockSize * s.numKvHeads;
        a.kRowStride = s.headDimK;
        a.kHeadStride = s.blockSize * s.headDimK;
        a.vRowStride = s.headDimV;
        a.vHeadStride = s.blockSize * s.headDimV;
    } else {
        a.blockRows = s.blockSize;
        a.kRowStride = static_cast<int64_t>(s.numKvHeads) * (s.headDimK - s.ropeDim);
        a.kHeadStride = s.headDimK - s.ropeDim;
        a.vRowStride = s.mlaCombined ? a.kRowStride : static_cast<int64_t>(s.numKvHeads) * s.headDimV;
        a.vHeadStride = s.mlaCombined ? s.headDimK - s.ropeDim : s.headDimV;
    }
    // (with per-sequence descale slices the attention kernel descales its partial rows itself)
    // With offsets (or under head compression, where the merge kernel cannot tell the descale slice) the attention
    // kernel descales its partial rows itself: added to a row already rounded to 16 bits, an offset that cancels
    // would magnify the rounding.
    a.finishV = (plan->useMfma && s.kvDtype == ATBMI_INT8 && s.descaleHeads == 0 && !s.hasOffset) ? 1 : 0;
    a.descaleHeads = s.kvDtype == ATBMI_INT8 ? s.descaleHeads : 0;
    a.razor = s.hasRazorOffset ? t->razorOffset : nullptr;
    if (s.hasMask) {
        a.mask = t->mask;
        a.maskBatchStride = s.maskBatchStride;
        a.maskHeadStride = s.maskHeadStride;
        a.maskLen = s.maskLen;
        a.maskVec = (reinterpret_cast<uintptr_t>(t->mask) % 8 == 0 && s.maskBatchStride % 4 == 0 &&
                     s.maskHeadStride % 4 == 0) ? 1 : 0;
    }
    a.logN = s.hasLogN ? t->logN : nullptr;
    a.scaleStride = s.descalePacked ? 2 : 1; // little endian: the low half of each uint64 comes first
    a.maskRowStep = s.maskRowBy == ATBMI_PA_MASK_ROW_SEQUENCE ? 0 : 1;
    a.qRope = s.ropeDim ? t->queryRope : nullptr;
    a.kRope = s.ropeDim ? t->keyRopeCache : nullptr;
    a.ropeDim = s.ropeDim;
    a.ropeRowStride = static_cast<int64_t>(s.numKvHeads) * s.ropeDim;
    a.lse = t->lse;
    a.nzShift = s.kvLayout == ATBMI_PA_KV_FRACTAL_NZ ? __builtin_ctz(static_cast<unsigned>(s.blockSize)) : 0;

    TimedLaunch timed;
    if (mayAllocate) {
        rc = TimedLaunchBegin(stream, &timed);
        if (rc != OK) {
            return rc;
        }
    }
    const int numItems = static_cast<int>(plan->items.size());
    PaStreamPlan &sp = plan->stream;
    if (plan->useMfma) {
        sp.seqs = plan->streamInline ? nullptr : reinterpret_cast<const PaSeq *>(ws + plan->offItems);
        sp.firstSeq = plan->streamInline ? nullptr : reinterpret_cast<const uint16_t *>(ws + plan->offSeqs);
        rc = LaunchPaMfma(s, a, sp, stream);
    } else {
        rc = LaunchPaScalar(s, a, numItems, stream);
    }
    if (rc == OK) {
        rc = TimedLaunchKernelDone(stream, timed);
    }
    bool merged = false;
    if (rc == OK) {
        if (plan->useMfma) {
            merged = plan->streamNeedsReduce;
            rc = merged ? LaunchPaStreamReduce(s, a, sp, stream) : OK;
        } else {
            merged = !plan->reduceSeqs.empty();
            rc = LaunchPaReduce(s, a, static_cast<int>(plan->reduceSeqs.size()), stream);
        }
    }
    const int closed = TimedLaunchEnd(stream, timed, merged && rc == OK);
    return rc != OK ? rc : closed;
}

} // namespace

extern "C" int atbmi_pa_decode(AtbmiPaPlan *plan, const AtbmiPaTensors *t, void *workspace, uint64_t workspaceBytes,
                               void *streamHandle)
{
    if (!plan || !t) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: null argument");
    }
    if (plan->nonEmpty == 0) {
        return OK; // every sequence is empty: nothing is written
    }
    return DecodeImpl(plan, t, workspace, workspaceBytes, streamHandle, true);
}

extern "C" uint64_t atbmi_pa_static_scratch_bytes(void)
{
    return STATIC_SCRATCH_BYTES;
}

extern "C" int atbmi_pa_decode_static(AtbmiPaPlan *plan, const AtbmiPaTensors *t, void *streamHandle)
{
    if (!plan || !t) {
        return Fail(ERR_INVALID_PARAM, "pa_decode_static: null argument");
    }
    if (plan->nonEmpty == 0) {
        return OK;
    }
    if (plan->blobBytes != 0) {
        return Fail(ERR_INVALID_PARAM, "pa_decode_static: the plan's tables (%llu bytes) do not travel in the kernel "
                                       "arguments (MFMA kernel, at most %d passes and %d workgroup ranges); use "
                                       "atbmi_pa_decode", (unsigned long long)plan->blobBytes, PA_INLINE_SEQS,
                    PA_INLINE_RANGES);
    }
    if (plan->wsBytes > STATIC_SCRATCH_BYTES) {
        return Fail(ERR_INVALID_PARAM, "pa_decode_static: the plan needs %llu bytes of partial rows, the static scratch "
                                       "holds %llu; use atbmi_pa_decode with a workspace",
                    (unsigned long long)plan->wsBytes, (unsigned long long)STATIC_SCRATCH_BYTES);
    }
    void *ptr = nullptr;
    if (plan->wsBytes > 0) {
        const int rc = StaticScratch(&ptr);
        if (rc != OK) {
            return rc;
        }
    }
    // Nothing in the scratch has to start at zero: every partial row and log-sum-exp the merge kernel
    // reads was written by the attention kernel of the same call.
    return DecodeImpl(plan, t, ptr, plan->wsBytes, streamHandle, false);
}

extern "C" int atbmi_timing_enable(int32_t enable)
{
    std::lock_guard<std::mutex> lock(g_timingMutex);
    g_timingEvery = enable > 0 ? enable : 0;
    g_timingLaunch = 0;
    return OK;
}

extern "C" int atbmi_timing_whole_calls(int32_t whole)
{
    std::lock_guard<std::mutex> lock(g_timingMutex);
    g_timingWhole = whole != 0;
    return OK;
}

extern "C" int atbmi_timing_read_samples(float *kernelMs, float *withMergeMs, int64_t capacity, int64_t *launches)
{
    std::vector<TimingRecord> records;
    {
        std::lock_guard<std::mutex> lock(g_timingMutex);
        records.swap(g_timingRecords);
    }
    int64_t count = 0;
    for (const TimingRecord &r : records) {
        hipEvent_t last = r.merged ? r.merged : r.end;
        ATBMI_HIP_CHECK(hipEventSynchronize(last));
        float ms = 0.0f, msMerged = 0.0f;
        ATBMI_HIP_CHECK(hipEventElapsedTime(&ms, r.begin, r.end));
        ATBMI_HIP_CHECK(hipEventElapsedTime(&msMerged, r.begin, last));
        if (count < capacity) {
            if (kernelMs) {
                kernelMs[count] = ms;
            }
            if (withMergeMs) {
                withMergeMs[count] = msMerged;
            }
            ++count;
        }
        (void)hipEventDestroy(r.begin);
        (void)hipEventDestroy(r.end);
        if (r.merged) {
            (void)hipEventDestroy(r.merged);
        }
    }
    if (launches) {
        *launches = count;
    }
    return OK;
}

extern "C" int atbmi_timing_read_split(double *kernelMs, double *withMergeMs, int64_t *launches)
{
    std::vector<float> kernel, merged;
    size_t pending = 0;
    {
        std::lock_guard<std::mutex> lock(g_timingMutex);
        pending = g_timingRecords.size();
    }
    try {
        kernel.resize(pending);
        merged.resize(pending);
    } catch (const std::bad_alloc &) {
        return Fail(ERR_OUT_OF_HOST_MEMORY, "timing_read: out of host memory");
    }
    int64_t count = 0;
    const int rc = atbmi_timing_read_samples(kernel.data(), merged.data(), static_cast<int64_t>(pending), &count);
    if (rc != OK) {
        return rc;
    }
    double sum = 0.0, sumMerged = 0.0;
    for (int64_t i = 0; i < count; ++i) {
        sum += kernel[static_cast<size_t>(i)];
        sumMerged += merged[static_cast<size_t>(i)];
    }
    if (kernelMs) {
        *kernelMs = sum;
    }
    if (withMergeMs) {
        *withMergeMs = sumMerged;
    }
    if (launches) {
        *launches = count;
    }
    return OK;
}

extern "C" int atbmi_timing_read(double *totalMs, int64_t *launches)
{
    return atbmi_timing_read_split(totalMs, nullptr, launches);
}
