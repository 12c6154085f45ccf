// C-ABI entry points of the decode GEMV: argument checks and per-format dispatch.
#include "ql_host.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    bool q4k_gemv_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int32_t *d_sums,
                         int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st);
    bool q6k_gemv_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int32_t *d_sums,
                         int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st);
    bool iq3s_gemv_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int32_t *d_sums,
                          int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st);
    int gemv_group_launch(const char *fn, const llam_ql_proj *projs, int num, const void *d_q8, int M, int K,
                          int device_id, hipStream_t st);

    namespace
    {
        bool check_common(const char *fn, uint8_t fmt, const void *d_w, const void *d_q8, int M, int N, int K)
        {
            if (fmt != LLAM_FMT_Q4_K && fmt != LLAM_FMT_Q6_K && fmt != LLAM_FMT_IQ3_S)
                return fail(fn, "unsupported weight format id %d", (int)fmt);
            if (M < 1 || M > LLAM_QL_MAX_GEMV_M)
                return fail(fn, "M=%d outside 1..%d", M, LLAM_QL_MAX_GEMV_M);
            if (N < 1 || K < 1)
                return fail(fn, "empty matrix (N=%d K=%d)", N, K);
            if ((K % 256) != 0)
                return fail(fn, "K must be a multiple of 256 (N=%d K=%d)", N, K);
            if (!d_w || !d_q8)
                return fail(fn, "null pointer");
            if (!aligned16(d_w) || !aligned4(d_q8))
                return fail(fn, "d_w must be 16-byte and d_q8 4-byte aligned");
            return true;
        }

        bool dispatch(const char *fn, uint8_t fmt, const void *d_w, const void *d_q8, float *d_y, int32_t *d_sums,
                      int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st)
        {
            switch (fmt)
            {
            case LLAM_FMT_Q4_K:
                return q4k_gemv_launch(fn, d_w, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
            case LLAM_FMT_Q6_K:
                return q6k_gemv_launch(fn, d_w, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
            default:
                return iq3s_gemv_launch(fn, d_w, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
            }
        }
    } // namespace
} // namespace llamql

extern "C" bool llam_ql_gemv(uint8_t fmt, const void *d_w, const void *d_q8, float *d_y,
                             int M, int N, int K, int ldy, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv";
    if (!check_common(fn, fmt, d_w, d_q8, M, N, K))
        return false;
    if (!d_y)
        return fail(fn, "null output");
    if (ldy < N)
        return fail(fn, "ldy=%d smaller than N=%d", ldy, N);
    if (!set_device(fn, device_id))
        return false;
    return dispatch(fn, fmt, d_w, d_q8, d_y, nullptr, M, N, K, ldy, 0, 0, device_id, as_stream(stream));
}

extern "C" bool llam_ql_gemv_fused(const llam_ql_proj *projs, int num, const void *d_q8,
                                   int M, int K, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_fused";
    if (num < 0 || num > LLAM_QL_MAX_FUSED)
        return fail(fn, "num=%d outside 0..%d", num, LLAM_QL_MAX_FUSED);
    if (num > 0 && !projs)
        return fail(fn, "null projection table");
    for (int i = 0; i < num; ++i)
    {
        if (!check_common(fn, projs[i].fmt, projs[i].d_w, d_q8, M, projs[i].N, K))
            return false;
        if (!projs[i].d_y || projs[i].ldy < projs[i].N)
            return fail(fn, "projection %d: bad output (ldy=%d N=%d)", i, projs[i].ldy, projs[i].N);
    }
    if (num == 0)
        return true;
    if (!set_device(fn, device_id))
        return false;
    // One quantised input.  Neighbouring projections of one format share a launch where
    // the kernel allows it (each keeps the row partition of its own launch, so the results
    // are those of separate calls); the rest are enqueued back to back on the same stream.
    for (int i = 0; i < num;)
    {
        const int took = gemv_group_launch(fn, projs + i, num - i, d_q8, M, K, device_id, as_stream(stream));
        if (took < 0)
            return false;
        if (took > 0)
        {
            i += took;
            continue;
        }
        if (!dispatch(fn, projs[i].fmt, projs[i].d_w, d_q8, projs[i].d_y, nullptr, M, projs[i].N, K,
                      projs[i].ldy, 0, 0, device_id, as_stream(stream)))
            return false;
        ++i;
    }
    return true;
}

extern "C" bool llam_ql_gemv_block_sums(uint8_t fmt, const void *d_w, const void *d_q8,
                                        int32_t *d_sums, int M, int N, int K, int row0,
                                        int nrows, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_block_sums";
    if (!check_common(fn, fmt, d_w, d_q8, M, N, K))
        return false;
    if (!d_sums)
        return fail(fn, "null output");
    if (row0 < 0 || nrows < 1 || (long)row0 + nrows > N)
        return fail(fn, "row window [%d,%d) outside [0,%d)", row0, row0 + nrows, N);
    if (!set_device(fn, device_id))
        return false;
    return dispatch(fn, fmt, d_w, d_q8, nullptr, d_sums, M, N, K, 0, row0, nrows, device_id, as_stream(stream));
}
