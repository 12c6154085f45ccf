// Decode GEMV launchers: one instantiation of the shared skeleton per weight format.
#include "gemv_traits_all.h"
#include "gemv_fast.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    bool q4k_gemv_launch(const char *fn, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                         int32_t *d_sums, int M, int N, int K, int ldy, int row0, int nrows, int device_id,
                         hipStream_t st)
    {
        return gemv_launch<Q4KTraits>(fn, d_w, d_plane, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
    }

    bool q6k_gemv_launch(const char *fn, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                         int32_t *d_sums, int M, int N, int K, int ldy, int row0, int nrows, int device_id,
                         hipStream_t st)
    {
        return gemv_launch<Q6KTraits>(fn, d_w, d_plane, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
    }

    bool iq3s_gemv_launch(const char *fn, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                         int32_t *d_sums, int M, int N, int K, int ldy, int row0, int nrows, int device_id,
                         hipStream_t st)
    {
        return gemv_launch<IQ3STraits>(fn, d_w, d_plane, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
    }

    namespace
    {
        template <class F>
        void describe(int M, int N, int K, bool has_plane, int device_id, llam_ql_gemv_plan *out)
        {
            // a batch the caller's batch plane serves runs on the matrix-unit plane kernel whatever
            // the plan for the matrix alone says
            if (has_plane && batch_plane_usable<F>(M, N, K))
            {
                out->kernel = GEMV_KERNEL_MFMA;
                out->m_first = M;
                out->slice_sb = K / 256;
                out->rows_per_wave = 0;
                out->decode_equivalent = 0;
                return;
            }
            const GemvPlan p = gemv_plan<F>(M, N, K, device_id);
            out->kernel = p.kernel;
            out->m_first = p.m_first;
            out->slice_sb = p.slice_sb;
            out->rows_per_wave = p.rows_per_wave;
            out->decode_equivalent = gemv_decode_equivalent<F>(M, N, K, device_id) ? 1 : 0;
        }
    } // namespace

    void gemv_describe(uint8_t fmt, int M, int N, int K, bool has_plane, int device_id, llam_ql_gemv_plan *out)
    {
        switch (fmt)
        {
        case LLAM_FMT_Q4_K: describe<Q4KTraits>(M, N, K, has_plane, device_id, out); break;
        case LLAM_FMT_Q6_K: describe<Q6KTraits>(M, N, K, has_plane, device_id, out); break;
        default: describe<IQ3STraits>(M, N, K, has_plane, device_id, out); break;
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
                if (mfma_eligible<F>(M, projs[0].N, K) || batch_plane_for<F>(projs[0].d_plane, M, projs[0].N, K))
                {
                    // .. unless a run of small matrices for the quad-lane kernel follows a Q4_K one (Q, then K
                    // and V): those share its launch
                    if constexpr (std::is_same<F, Q4KTraits>::value)
                        if (src.kind == ACT_SRC_Q8 && gemv_mfma_quad_ok(M, projs[0].N, K, device_id))
                        {
                            QuadProj pr[QUAD_MAX_PROJ];
                            int na = 0, nb = 0;
                            auto quad_only = [&](auto tag, const llam_ql_proj &q) {
                                typedef decltype(tag) G;
                                return quad_eligible<G>(M, q.N, K) && !mfma_eligible<G>(M, q.N, K) &&
                                       !batch_plane_for<G>(q.d_plane, M, q.N, K);
                            };
                            while (1 + na < num && na < QUAD_MAX_PROJ && projs[1 + na].fmt == LLAM_FMT_Q4_K &&
                                   quad_only(Q4KTraits{}, projs[1 + na]))
                            {
                                pr[na] = QuadProj{projs[1 + na].d_w, projs[1 + na].d_y, projs[1 + na].N, projs[1 + na].ldy};
                                ++na;
                            }
                            while (1 + na + nb < num && na + nb < QUAD_MAX_PROJ && projs[1 + na + nb].fmt == LLAM_FMT_Q6_K &&
                                   quad_only(Q6KTraits{}, projs[1 + na + nb]))
                            {
                                pr[na + nb] = QuadProj{projs[1 + na + nb].d_w, projs[1 + na + nb].d_y, projs[1 + na + nb].N,
                                                       projs[1 + na + nb].ldy};
                                ++nb;
                            }
                            if (na + nb > 0 && quad_lds_bytes(M, K / 256) <= QUAD_MAX_LDS)
                                return gemv_mfma_quad_launch(fn, projs[0].d_w,
                                                             batch_plane_for<F>(projs[0].d_plane, M, projs[0].N, K),
                                                             projs[0].d_y, projs[0].N, projs[0].ldy, pr, na, nb, src.q8, M, K,
                                                             device_id, st)
                                           ? 1 + na + nb
                                           : -1;
                        }
                    return gemv_mfma_launch<F>(fn, projs[0].d_w, batch_plane_for<F>(projs[0].d_plane, M, projs[0].N, K), src,
                                                projs[0].d_y, M, projs[0].N, K, projs[0].ldy, device_id, st)
                               ? 1
                               : -1;
                }
            QuadProj pr[QUAD_MAX_PROJ];
            int n = 0;
            while (n < num && n < QUAD_MAX_PROJ && projs[n].fmt == projs[0].fmt &&
                   quad_eligible<F>(M, projs[n].N, K) && !mfma_eligible<F>(M, projs[n].N, K) &&
                   !batch_plane_for<F>(projs[n].d_plane, M, projs[n].N, K))
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
                           quad_eligible<G>(M, projs[n + nb].N, K) && !mfma_eligible<G>(M, projs[n + nb].N, K) &&
                           !batch_plane_for<G>(projs[n + nb].d_plane, M, projs[n + nb].N, K))
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

// ---- the Q6_K batch plane ---------------------------------------------------------------------
namespace llamql
{
    // Thread (row, super-block, block j, half h) writes the 16 requantised elements 16h..16h+15 of
    // block j of the row -- what lane (row, h) of gemv_mfma_q6k_kernel hands the matrix unit --
    // and, for h = 0, the block's scale.  Rows past N (the last group's padding) are zeros.
    __global__ void __launch_bounds__(256) build_q6k_plane_kernel(const uint8_t *prepared, uint8_t *plane, long N, int nsb)
    {
        const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
        const size_t rows = q6k_plane_groups(N) * 4;
        if (idx >= rows * (size_t)nsb * 16)
            return;
        const int h = (int)(idx & 1), j = (int)((idx >> 1) & 7);
        const size_t rs = idx >> 4; // row * nsb + sb
        const size_t row = rs / (size_t)nsb;
        const int sb = (int)(rs - row * (size_t)nsb);
        const size_t cell = (row >> 2) * (size_t)nsb + (size_t)sb; // the group's super-block
        v4i *dst = reinterpret_cast<v4i *>(plane + (cell * 8 + (size_t)j) * 128 + (row & 3) * 32 + 16 * h);
        uint16_t *dsc = reinterpret_cast<uint16_t *>(plane + q6k_plane_scales_offset(N, nsb) + cell * 64 + (row & 3) * 16) + j;
        if ((long)row >= N)
        {
            *dst = (v4i){0, 0, 0, 0};
            if (h == 0)
                *dsc = 0;
            return;
        }
        const size_t T = (size_t)N * (size_t)nsb, t = row * (size_t)nsb + (size_t)sb;
        const int n = j >> 2, s = j & 3;
        const v4i lo = *reinterpret_cast<const v4i *>(prepared + t * 128 + 64 * n + 32 * (s & 1) + 16 * h);
        const v4i hi = *reinterpret_cast<const v4i *>(prepared + T * 128 + t * 64 + 32 * n + 16 * h);
        const uint32_t rec = *reinterpret_cast<const uint32_t *>(prepared + q6k_factors_offset(T) + t * 32 + 4 * q6k_code_pos(j));
        int f;
        float bscale;
        q6k_block_factor(rec, h ? Q6K_CODE_BIG1 : 0u, f, bscale);
        const unsigned short fu = (unsigned short)f, ku = (unsigned short)(128 - 32 * f);
        const Q6KQuad::v2s ff = {fu, fu}, cc = {ku, ku};
        const uint32_t k4 = 0x0F0F0F0Fu, k2 = 0x03030303u;
        auto q4 = [&](int l, int hq) {
            const uint32_t nib = (s >= 2 ? (uint32_t)l >> 4 : (uint32_t)l) & k4;
            const uint32_t q = nib | ((((uint32_t)hq >> (2 * s)) & k2) << 4);
            return Q6KQuad::requant4(q, ff, cc);
        };
        *dst = (v4i){q4(lo.x, hi.x), q4(lo.y, hi.y), q4(lo.z, hi.z), q4(lo.w, hi.w)};
        if (h == 0)
            *dsc = (uint16_t)(rec >> 16);
    }

    // One thread per 16-byte piece of a super-block: piece 0, the head, goes to the heads plane,
    // piece 1 + 2c + h is half h of group c.  Rows past N (the last group's padding) are zeros.
    __global__ void __launch_bounds__(256) build_q4k_plane_kernel(const uint8_t *prepared, uint8_t *plane, long N, int nsb)
    {
        const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
        const size_t rows = q6k_plane_groups(N) * 4;
        if (idx >= rows * (size_t)nsb * 9)
            return;
        const size_t rs = idx / 9; // row * nsb + sb
        const int piece = (int)(idx - rs * 9);
        const size_t row = rs / (size_t)nsb;
        const int sb = (int)(rs - row * (size_t)nsb);
        const size_t cell = (row >> 2) * (size_t)nsb + (size_t)sb; // the group's super-block
        v4i v = {0, 0, 0, 0};
        if ((long)row < N)
            v = *reinterpret_cast<const v4i *>(prepared + rs * 144 + piece * 16);
        uint8_t *dst = piece == 0 ? plane + q4k_plane_heads_offset(N, nsb) + cell * 64 + (row & 3) * 16
                                  : plane + (cell * 4 + (size_t)((piece - 1) >> 1)) * 128 + (row & 3) * 32 + 16 * ((piece - 1) & 1);
        *reinterpret_cast<v4i *>(dst) = v;
    }

    // A plane exists for Q6_K rows of eight super-blocks and more, and for the Q4_K shapes whose
    // batches of 5..8 go to the matrix-unit kernel.
    static bool batch_plane_shape(uint8_t fmt, int N, int K)
    {
        if (N < 1 || K < 2048 || K % 256 != 0)
            return false;
        // (the kernels' lane offsets are 32-bit)
        if (fmt == LLAM_FMT_Q6_K)
            return q6k_plane_bytes(N, K / 256) < ((size_t)1 << 32);
        if (fmt == LLAM_FMT_Q4_K)
            return mfma_eligible<Q4KTraits>(8, N, K) && q4k_plane_bytes(N, K / 256) < ((size_t)1 << 32);
        return false;
    }
    static size_t batch_plane_size(uint8_t fmt, int N, int K)
    {
        return fmt == LLAM_FMT_Q6_K ? q6k_plane_bytes(N, K / 256) : q4k_plane_bytes(N, K / 256);
    }
} // namespace llamql

extern "C" bool llam_ql_gemv_plane_split_supported(uint8_t fmt, int M, int N, int K)
{
    if (K < 1)
        return false;
    return fmt == LLAM_FMT_Q6_K ? llamql::gemv_mfma_q6k_split_ok(M, N, K)
                                : fmt == LLAM_FMT_Q4_K && llamql::gemv_mfma_q4k_split_ok(M, N, K);
}

extern "C" bool llam_ql_gemv_plane_split(uint8_t fmt, const void *d_plane, const void *d_q8, float *d_y_lo,
                                         float *d_y_hi, int M, int N, int K, int ldy, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_plane_split";
    if (!llam_ql_gemv_plane_split_supported(fmt, M, N, K))
        return fail(fn, "not served for format %d, M=%d, N=%d, K=%d (llam_ql_gemv_plane_split_supported)", (int)fmt, M, N, K);
    if (!d_plane || !d_q8 || !d_y_lo || !d_y_hi || d_y_lo == d_y_hi)
        return fail(fn, "null pointer, or one buffer for both halves");
    if (!aligned16(d_plane) || !aligned4(d_q8))
        return fail(fn, "d_plane must be 16-byte and d_q8 4-byte aligned");
    if (ldy < N)
        return fail(fn, "ldy=%d smaller than N=%d", ldy, N);
    if (!set_device(fn, device_id))
        return false;
    if (fmt == LLAM_FMT_Q4_K)
        return gemv_mfma_q4k_split_launch(fn, d_plane, d_q8, d_y_lo, d_y_hi, M, N, K, ldy, device_id, as_stream(stream));
    return gemv_mfma_q6k_split_launch(fn, d_plane, d_q8, d_y_lo, d_y_hi, M, N, K, ldy, device_id, as_stream(stream));
}

extern "C" bool llam_ql_gemv_gate_up_swiglu_supported(uint8_t fmt, int M, int N, int K)
{
    return fmt == LLAM_FMT_Q4_K && M >= 1 && M <= LLAM_QL_MAX_GEMV_M && N >= 1 && K >= 1 &&
           llamql::gemv_mfma_q4k_swiglu_ok(M, N, K);
}

extern "C" bool llam_ql_gemv_gate_up_swiglu(uint8_t fmt, const void *d_w_gate, const void *d_plane_gate,
                                            const void *d_w_up, const void *d_plane_up, const void *d_q8,
                                            float *d_y_gate, float *d_y_up, int ldy, void *d_q8_out, int M, int N,
                                            int K, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_gate_up_swiglu";
    if (!llam_ql_gemv_gate_up_swiglu_supported(fmt, M, N, K))
        return fail(fn, "not served for format %d, M=%d, N=%d, K=%d (llam_ql_gemv_gate_up_swiglu_supported)", (int)fmt, M,
                    N, K);
    if (!d_w_gate || !d_w_up || !d_q8 || !d_q8_out)
        return fail(fn, "null pointer");
    if (!aligned16(d_w_gate) || !aligned16(d_w_up) || !aligned4(d_q8) || !aligned4(d_q8_out))
        return fail(fn, "the matrices must be 16-byte, the Q8_1 buffers 4-byte aligned");
    if ((d_plane_gate == nullptr) != (d_plane_up == nullptr))
        return fail(fn, "batch planes for both matrices or for neither");
    if (d_plane_gate && (!aligned16(d_plane_gate) || !aligned16(d_plane_up) || llam_ql_batch_plane_bytes(fmt, N, K) == 0))
        return fail(fn, "the planes must be 16-byte aligned and of a shape that has one (llam_ql_batch_plane_bytes)");
    if ((d_y_gate || d_y_up) && ldy < N)
        return fail(fn, "ldy=%d smaller than N=%d", ldy, N);
    if (!set_device(fn, device_id))
        return false;
    return gemv_mfma_q4k_swiglu_launch(fn, d_w_gate, d_plane_gate, d_w_up, d_plane_up, d_q8, d_y_gate, d_y_up, ldy,
                                       d_q8_out, M, N, K, device_id, as_stream(stream));
}

extern "C" size_t llam_ql_batch_plane_bytes(uint8_t fmt, int N, int K)
{
    return llamql::batch_plane_shape(fmt, N, K) ? llamql::batch_plane_size(fmt, N, K) : 0;
}

extern "C" bool llam_ql_build_batch_plane(uint8_t fmt, const void *d_prepared, void *d_plane, int N, int K,
                                          int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_build_batch_plane";
    if (!batch_plane_shape(fmt, N, K))
        return fail(fn, "no batch plane for format %d, N=%d, K=%d (llam_ql_batch_plane_bytes is 0)", (int)fmt, N, K);
    if (!d_prepared || !d_plane)
        return fail(fn, "null pointer");
    if (!aligned16(d_prepared) || !aligned16(d_plane))
        return fail(fn, "d_prepared and d_plane must be 16-byte aligned");
    if (!set_device(fn, device_id))
        return false;
    const int nsb = K / 256;
    const size_t items = q6k_plane_groups(N) * 4 * (size_t)nsb * (fmt == LLAM_FMT_Q6_K ? 16 : 9);
    const size_t grid = (items + 255) / 256;
    if (grid > 0x7FFFFFFFull)
        return fail(fn, "matrix too large (N=%d K=%d)", N, K);
    if (fmt == LLAM_FMT_Q6_K)
        hipLaunchKernelGGL(build_q6k_plane_kernel, dim3((unsigned)grid), dim3(256), 0, as_stream(stream),
                           static_cast<const uint8_t *>(d_prepared), static_cast<uint8_t *>(d_plane), (long)N, nsb);
    else
        hipLaunchKernelGGL(build_q4k_plane_kernel, dim3((unsigned)grid), dim3(256), 0, as_stream(stream),
                           static_cast<const uint8_t *>(d_prepared), static_cast<uint8_t *>(d_plane), (long)N, nsb);
    return launched(fn);
}
