// MultiLatentAttention, maskType MASK_TYPE_MASK_FREE with several query tokens (decode): the compressed mask the
// caller hands over, a template [rows, 128] (or one per sequence, [batch, rows, 128]) with rows = 125 + 2 q for q
// query tokens, is turned into one mask row per query token, [numQueryRows, maskLen], which the decode kernels
// then add to the scores like a MASK_TYPE_SPEC mask.
//
// What the reference's kernel reads of the template (src/kernels/mixkernels/multi_latent_attention/op_kernel/
// mla.cce:3719-3750 with 2581-2592, tiles of 128 tokens): for a sequence of k tokens whose last tile holds
// n = k - 128 L tokens (L = (k - 1) / 128), query token i of q takes
//   in the last tile          template row n - 1 + i, column = token - 128 L;
//   in the tile before it     template row n + 127 + i, column = token - 128 (L - 1), and only when n < q - 1
//                             (the look-ahead triangle then reaches back into that tile);
//   nothing anywhere else.
// With the template of the reference's tests (-10000 where column - row >= 2 - q,
// tests/apitest/opstest/python/operations/multi_latent_attention/test_multi_latent_attention_mtp.py:342-358) that
// is the causal triangle over the last q tokens. Template rows the tensor does not have read as 0.
#include <vector>
#include "pa_internal.h"
#include "upload_ring.h"

namespace atbmi {
namespace maskfree {

constexpr int TILE = 128;
constexpr int THREADS = 256;

struct Row {
    int32_t seq;     // index into the template's batch dimension
    int32_t ctxLen;  // k
    int32_t queries; // q
    int32_t index;   // i
};

struct Args {
    const uint16_t *mask; // the template
    uint16_t *out;        // [numRows, maskLen]
    const Row *rows;
    int64_t batchStride;  // elements between the templates of two sequences (0: one template)
    int32_t templateRows;
    int32_t maskLen;
};

__global__ __launch_bounds__(THREADS) void MaskFreeExpandKernel(const Args a)
{
    const Row r = a.rows[blockIdx.y];
    const int j = blockIdx.x * THREADS + threadIdx.x;
    if (j >= a.maskLen) {
        return;
    }
    uint16_t v = 0;
    if (j < r.ctxLen) {
        const int last = (r.ctxLen - 1) / TILE;
        const int n = r.ctxLen - last * TILE;
        const int tile = j / TILE;
        int row = -1;
        if (tile == last) {
            row = n - 1 + r.index;
        } else if (tile == last - 1 && n < r.queries - 1) {
            row = n + TILE - 1 + r.index;
        }
        if (row >= 0 && row < a.templateRows) {
            v = a.mask[r.seq * a.batchStride + static_cast<int64_t>(row) * TILE + j % TILE];
        }
    }
    a.out[static_cast<int64_t>(blockIdx.y) * a.maskLen + j] = v;
}

int BuildRows(const AtbmiMlaMaskFreeCall *c, std::vector<Row> *rows)
{
    if (!c || !c->hostContextLens || !c->hostQueryLens) {
        return Fail(ERR_INVALID_PARAM, "mla_mask_free: null call or length arrays");
    }
    if (c->batch <= 0 || c->templateRows <= 0 || c->maskLen <= 0 || c->numQueryRows < 0 ||
        (c->templateBatch != 0 && c->templateBatch != c->batch)) {
        return Fail(ERR_INVALID_PARAM, "mla_mask_free: batch %d, template [%d x] %d x 128, mask rows of %d, %d query rows",
                    c->batch, c->templateBatch, c->templateRows, c->maskLen, c->numQueryRows);
    }
    for (int32_t b = 0; b < c->batch; ++b) {
        const int32_t k = c->hostContextLens[b], q = c->hostQueryLens[b];
        if (k < 0 || q < 0 || k > c->maskLen || (k > 0 && q > k)) {
            return Fail(ERR_INVALID_PARAM, "mla_mask_free: sequence %d has context %d (mask rows of %d) and %d query tokens",
                        b, k, c->maskLen, q);
        }
        // (an empty context keeps its query rows, as in the decode plan of MultiLatentAttention: their mask rows are zeros)
        if (q > 1 && k > 0) {
            // the template must hold every row this sequence reads
            const int n = k - (k - 1) / TILE * TILE;
            const int top = (n < q - 1 && k > TILE ? n + TILE - 1 : n - 1) + q - 1;
            if (top >= c->templateRows) {
                return Fail(ERR_INVALID_PARAM, "mla_mask_free: sequence %d (context %d, %d query tokens) reads template "
                                               "row %d, the template has %d", b, k, q, top, c->templateRows);
            }
        }
        for (int32_t i = 0; i < q; ++i) {
            if (rows) {
                rows->push_back(Row{c->templateBatch ? b : 0, k, q, i});
            }
        }
    }
    return OK;
}

} // namespace maskfree
} // namespace atbmi

using namespace atbmi;

extern "C" int atbmi_mla_mask_free_workspace_size(const AtbmiMlaMaskFreeCall *call, uint64_t *bytes)
{
    if (!bytes) {
        return Fail(ERR_INVALID_PARAM, "mla_mask_free_workspace_size: null result pointer");
    }
    std::vector<maskfree::Row> rows;
    const int rc = maskfree::BuildRows(call, &rows);
    if (rc != OK) {
        return rc;
    }
    if (static_cast<int64_t>(rows.size()) > call->numQueryRows) {
        return Fail(ERR_INVALID_PARAM, "mla_mask_free: the lengths ask for %lld query rows, the mask holds %d",
                    (long long)rows.size(), call->numQueryRows);
    }
    *bytes = rows.size() * sizeof(maskfree::Row);
    return OK;
}

extern "C" int atbmi_mla_mask_free_expand(const AtbmiMlaMaskFreeCall *call, void *workspaceDevice, uint64_t workspaceBytes,
                                          void *stream)
{
    std::vector<maskfree::Row> rows;
    int rc = maskfree::BuildRows(call, &rows);
    if (rc != OK) {
        return rc;
    }
    if (rows.empty()) {
        return OK;
    }
    if (static_cast<int64_t>(rows.size()) > call->numQueryRows || rows.size() > 65535) {
        return Fail(ERR_INVALID_PARAM, "mla_mask_free: %lld query rows (the mask holds %d; at most 65535 a call)",
                    (long long)rows.size(), call->numQueryRows);
    }
    if (!call->maskTemplate || !call->outMask) {
        return Fail(ERR_INVALID_PARAM, "mla_mask_free: null tensor pointer");
    }
    const size_t bytes = rows.size() * sizeof(maskfree::Row);
    if (!workspaceDevice || workspaceBytes < bytes) {
        return Fail(ERR_INVALID_PARAM, "mla_mask_free: workspace of %llu bytes, %llu needed", (unsigned long long)workspaceBytes,
                    (unsigned long long)bytes);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    rc = UploadTable(rows.data(), bytes, workspaceDevice, s);
    if (rc != OK) {
        return rc;
    }
    maskfree::Args a{};
    a.mask = static_cast<const uint16_t *>(call->maskTemplate);
    a.out = static_cast<uint16_t *>(call->outMask);
    a.rows = static_cast<const maskfree::Row *>(workspaceDevice);
    a.batchStride = call->templateBatch ? static_cast<int64_t>(call->templateRows) * maskfree::TILE : 0;
    a.templateRows = call->templateRows;
    a.maskLen = call->maskLen;
    const dim3 grid((call->maskLen + maskfree::THREADS - 1) / maskfree::THREADS, static_cast<unsigned>(rows.size()));
    maskfree::MaskFreeExpandKernel<<<grid, maskfree::THREADS, 0, s>>>(a);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}
