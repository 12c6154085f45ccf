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

    namespace
    {
        template <class F>
        void describe(int M, int N, int K, int device_id, llam_ql_gemv_plan *out)
        {
            const GemvPlan p = gemv_plan<F>(M, N, K, device_id);
            out->kernel = p.kernel;
            out->m_first = p.m_first;
            out->slice_sb = p.slice_sb;
            out->rows_per_wave = p.rows_per_wave;
            out->decode_equivalent = gemv_decode_equivalent<F>(M, N, K, device_id) ? 1 : 0;
        }
    } // namespace

    void gemv_describe(uint8_t fmt, int M, int N, int K, int device_id, llam_ql_gemv_plan *out)
    {
        switch (fmt)
        {
        case LLAM_FMT_Q4_K: describe<Q4KTraits>(M, N, K, device_id, out); break;
        case LLAM_FMT_Q6_K: describe<Q6KTraits>(M, N, K, device_id, out); break;
        default: describe<IQ3STraits>(M, N, K, device_id, out); break;
        }
    }

    namespace
    {
        // the format that can share a quad-lane launch with F (Q and K in Q4_K with V in Q6_K)
        template <class F>
        struct Other
        {
            static constexpr bool exists = false;
        };
        template <>
        struct Other<Q4KTraits>
        {
            static constexpr bool exists = true;
            typedef Q6KTraits type;
            static constexpr uint8_t fmt = LLAM_FMT_Q6_K;
        };
        template <>
        struct Other<Q6KTraits>
        {
            static constexpr bool exists = true;
            typedef Q4KTraits type;
            static constexpr uint8_t fmt = LLAM_FMT_Q4_K;
        };

        template <class F>
        int group_launch(const char *fn, const llam_ql_proj *projs, int num, const ActSource &src, int M, int K,
                         int device_id, hipStream_t st)
        {
            // batches that go to the matrix-unit kernel launch one matrix at a time
            if constexpr (F::USE_MFMA_BATCH)
                if (mfma_eligible<F>(M, projs[0].N, K))
                    return gemv_mfma_launch<F>(fn, projs[0].d_w, src, projs[0].d_y, M, projs[0].N, K, projs[0].ldy,
                                                device_id, st)
                               ? 1
                               : -1;
            QuadProj pr[QUAD_MAX_PROJ];
            int n = 0;
            while (n < num && n < QUAD_MAX_PROJ && projs[n].fmt == projs[0].fmt &&
                   quad_eligible<F>(M, projs[n].N, K) && !mfma_eligible<F>(M, projs[n].N, K))
            {
                pr[n] = QuadProj{projs[n].d_w, projs[n].d_y, projs[n].N, projs[n].ldy};
                ++n;
            }
            // a following run in the other quad-lane format joins the launch (Q and K with V)
            if constexpr (F::USE_QUAD && Other<F>::exists)
                if (n >= 1 && n < QUAD_MAX_PROJ && src.kind != ACT_SRC_SWIGLU)
                {
                    typedef typename Other<F>::type G;
                    int nb = 0;
                    while (n + nb < num && n + nb < QUAD_MAX_PROJ && projs[n + nb].fmt == Other<F>::fmt &&
                           quad_eligible<G>(M, projs[n + nb].N, K) && !mfma_eligible<G>(M, projs[n + nb].N, K))
                    {
                        pr[n + nb] = QuadProj{projs[n + nb].d_w, projs[n + nb].d_y, projs[n + nb].N, projs[n + nb].ldy};
                        ++nb;
                    }
                    if (nb > 0)
                        return gemv_quad_dual<F, G>(fn, pr, n, nb, src, M, K, device_id, st) ? n + nb : -1;
                }
            // a single matrix on Q8_1 input goes through the general launcher
            if (n < (src.kind == ACT_SRC_Q8 ? 2 : 1))
                return 0;
            return gemv_quad_multi<F>(fn, pr, n, src, M, K, device_id, st) ? n : -1;
        }
    } // namespace

    // Whether a projection of this shape can take its activations from the norm fused into the
    // quad-lane kernel (ACT_SRC_RMSNORM).
    bool gemv_norm_fusable(uint8_t fmt, int M, int N, int K)
    {
        if (M < 1 || M > QUAD_NORM_MAX_M)
            return false;
        switch (fmt)
        {
        case LLAM_FMT_Q4_K: return quad_eligible<Q4KTraits>(M, N, K) && quad_lds_bytes(M, K / 256) + QUAD_NORM_LDS <= QUAD_MAX_LDS;
        case LLAM_FMT_Q6_K: return quad_eligible<Q6KTraits>(M, N, K) && quad_lds_bytes(M, K / 256) + QUAD_NORM_LDS <= QUAD_MAX_LDS;
        case LLAM_FMT_IQ3_S:
            return quad_eligible<IQ3STraits>(M, N, K) &&
                   quad_lds_bytes(M, K / 256) + QUAD_NORM_LDS + IQ3STraits::Quad::STATIC_LDS <= QUAD_MAX_LDS;
        default: return false;
        }
    }

    namespace
    {
        template <class F>
        bool accumulate_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int M, int N, int K,
                               int ldy, int device_id, hipStream_t st, bool query)
        {
            const GemvPlan p = gemv_plan<F>(M, N, K, device_id);
            if (p.kernel != GEMV_KERNEL_QUAD || p.m_first < M)
                return query ? false : fail(fn, "M=%d N=%d K=%d: not a single quad-lane launch", M, N, K);
            const QuadProj pr{d_w, d_y, N, ldy};
            return gemv_quad_multi<F>(fn, &pr, 1, act_source_q8(d_q8), M, K, device_id, st, nullptr, 0, 0,
                                      query ? QUAD_ACC_QUERY : QUAD_ACC_LAUNCH);
        }
    } // namespace

    // y += W a in the GEMV's own launch (query: only whether the shape's launch can do that).
    bool gemv_accumulate(const char *fn, uint8_t fmt, const void *d_w, const void *d_q8, float *d_y, int M, int N,
                         int K, int ldy, int device_id, hipStream_t st, bool query)
    {
        switch (fmt)
        {
        case LLAM_FMT_Q4_K: return accumulate_launch<Q4KTraits>(fn, d_w, d_q8, d_y, M, N, K, ldy, device_id, st, query);
        case LLAM_FMT_Q6_K: return accumulate_launch<Q6KTraits>(fn, d_w, d_q8, d_y, M, N, K, ldy, device_id, st, query);
        case LLAM_FMT_IQ3_S: return accumulate_launch<IQ3STraits>(fn, d_w, d_q8, d_y, M, N, K, ldy, device_id, st, query);
        default: return false;
        }
    }

    // Launches the longest run of projections at the head of `projs` (same format, all fit
    // for the quad-lane kernel) as ONE kernel.  Returns how many it covered, 0 when the
    // first projection has to go through its own launch on Q8_1 input, -1 on error.
    int gemv_group_launch(const char *fn, const llam_ql_proj *projs, int num, const ActSource &src, int M, int K,
                          int device_id, hipStream_t st)
    {
        if (num < 1)
            return 0;
        switch (projs[0].fmt)
        {
        case LLAM_FMT_Q4_K: return group_launch<Q4KTraits>(fn, projs, num, src, M, K, device_id, st);
        case LLAM_FMT_Q6_K: return group_launch<Q6KTraits>(fn, projs, num, src, M, K, device_id, st);
        case LLAM_FMT_IQ3_S: return group_launch<IQ3STraits>(fn, projs, num, src, M, K, device_id, st);
        default: return 0;
        }
    }
} // namespace llamql
