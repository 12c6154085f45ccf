// Decode GEMV launchers: one instantiation of the shared skeleton per weight format.
#include "gemv_traits_all.h"
#include "gemv_fast.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    bool q4k_gemv_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int32_t *d_sums,
                         int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st)
    {
        return gemv_launch<Q4KTraits>(fn, d_w, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
    }

    bool q6k_gemv_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int32_t *d_sums,
                         int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st)
    {
        return gemv_launch<Q6KTraits>(fn, d_w, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
    }

    bool iq3s_gemv_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int32_t *d_sums,
                          int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st)
    {
        return gemv_launch<IQ3STraits>(fn, d_w, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
    }
} // namespace llamql
