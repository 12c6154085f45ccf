// C-ABI entry points of the decode GEMV: argument checks and per-format dispatch.
#include "ql_host.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    bool q4k_gemv_launch(const char *fn, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                         int32_t *d_sums, int M, int N, int K, int ldy, int row0, int nrows, int device_id,
                         hipStream_t st);
    bool q6k_gemv_launch(const char *fn, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                         int32_t *d_sums, int M, int N, int K, int ldy, int row0, int nrows, int device_id,
                         hipStream_t st);
    bool iq3s_gemv_launch(const char *fn, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                          int32_t *d_sums, int M, int N, int K, int ldy, int row0, int nrows, int device_id,
                          hipStream_t st);
    void gemv_describe(uint8_t fmt, int M, int N, int K, bool has_plane, int device_id, llam_ql_gemv_plan *out);
    bool gemv_norm_fusable(uint8_t fmt, int M, int N, int K);
    bool gemv_accumulate(const char *fn, uint8_t fmt, const void *d_w, const void *d_q8, float *d_y, int M, int N,
                         int K, int ldy, int device_id, hipStream_t st, bool query);
    int gemv_group_launch(const char *fn, const llam_ql_proj *projs, int num, const ActSource &src, int M, int K,
                          int device_id, hipStream_t st);

    namespace
    {
        bool check_matrix(const char *fn, uint8_t fmt, const void *d_w, int M, int N, int K)
        {
            if (fmt != LLAM_FMT_Q4_K && fmt != LLAM_FMT_Q6_K && fmt != LLAM_FMT_IQ3_S)
                return fail(fn, "unsupported weight format id %d", (int)fmt);
            if (M < 1 || M > LLAM_QL_MAX_GEMV_M)
                return fail(fn, "M=%d outside 1..%d", M, LLAM_QL_MAX_GEMV_M);
            if (N < 1 || K < 1)
                return fail(fn, "empty matrix (N=%d K=%d)", N, K);
            if ((K % 256) != 0)
                return fail(fn, "K must be a multiple of 256 (N=%d K=%d)", N, K);
            if (!d_w)
                return fail(fn, "null pointer");
            if (!aligned16(d_w))
                return fail(fn, "d_w must be 16-byte aligned");
            return true;
        }

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

        // A caller's batch plane must be one llam_ql_build_batch_plane can have filled for this matrix.
        bool check_plane(const char *fn, uint8_t fmt, const void *d_plane, int N, int K)
        {
            if (!d_plane)
                return true;
            if (!aligned16(d_plane))
                return fail(fn, "d_plane must be 16-byte aligned");
            if (llam_ql_batch_plane_bytes(fmt, N, K) == 0)
                return fail(fn, "format %d, N=%d, K=%d has no batch plane (llam_ql_batch_plane_bytes is 0)", (int)fmt, N, K);
            return true;
        }

        bool dispatch(const char *fn, uint8_t fmt, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                      int32_t *d_sums, int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st)
        {
            switch (fmt)
            {
            case LLAM_FMT_Q4_K:
                return q4k_gemv_launch(fn, d_w, d_plane, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
            case LLAM_FMT_Q6_K:
                return q6k_gemv_launch(fn, d_w, d_plane, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
            default:
                return iq3s_gemv_launch(fn, d_w, d_plane, d_q8, d_y, d_sums, M, N, K, ldy, row0, nrows, device_id, st);
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
    return dispatch(fn, fmt, d_w, nullptr, d_q8, d_y, nullptr, M, N, K, ldy, 0, 0, device_id, as_stream(stream));
}

extern "C" bool llam_ql_gemv_plane(uint8_t fmt, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                                   int M, int N, int K, int ldy, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_plane";
    if (!check_common(fn, fmt, d_w, d_q8, M, N, K) || !check_plane(fn, fmt, d_plane, N, K))
        return false;
    if (!d_y)
        return fail(fn, "null output");
    if (ldy < N)
        return fail(fn, "ldy=%d smaller than N=%d", ldy, N);
    if (!set_device(fn, device_id))
        return false;
    return dispatch(fn, fmt, d_w, d_plane, d_q8, d_y, nullptr, M, N, K, ldy, 0, 0, device_id, as_stream(stream));
}

namespace llamql
{
    namespace
    {
        // Projections of one input, in order.  Neighbouring projections of one format share a
        // launch where the kernel allows it (each keeps the row partition of its own launch,
        // so the results are those of separate calls); the rest are enqueued back to back on
        // the same stream.  fp32 input is quantised inside the kernels; for the first
        // projection whose kernel cannot do that it is quantised into d_q8_scratch, which
        // then serves the remaining projections.
        bool run_projections(const char *fn, const llam_ql_proj *projs, int num, ActSource src, int M, int K,
                             void *d_q8_scratch, int device_id, void *stream)
        {
            // Every workgroup of a self-quantising launch quantises all M*K activations again.
            // Measured against a quantiser launch of its own (about 4.5 us) that pays off for a
            // single short row; beyond it the scratch buffer, when there is one, is used.
            const bool self_quantise =
                src.kind == ACT_SRC_Q8 || !d_q8_scratch || (src.kind == ACT_SRC_F32 && (long)M * K <= 6144);
            for (int i = 0; i < num;)
            {
                const int took = (self_quantise || src.kind == ACT_SRC_Q8)
                                     ? gemv_group_launch(fn, projs + i, num - i, src, M, K, device_id,
                                                         as_stream(stream))
                                     : 0;
                if (took < 0)
                    return false;
                if (took > 0)
                {
                    i += took;
                    continue;
                }
                if (src.kind != ACT_SRC_Q8)
                {
                    if (!d_q8_scratch)
                        return fail(fn, "projection %d (format %d, N=%d, K=%d) needs d_q8_scratch", i,
                                    (int)projs[i].fmt, projs[i].N, K);
                    const size_t row_bytes = (size_t)(K / 32) * sizeof(llam_block_q8_1);
                    const int rows_per_call = src.ldx == K ? M : 1;
                    for (int m = 0; m < M; m += rows_per_call)
                    {
                        void *dst = static_cast<uint8_t *>(d_q8_scratch) + (size_t)m * row_bytes;
                        const float *x = src.x + (size_t)m * src.ldx;
                        const bool ok = src.kind == ACT_SRC_F32
                                            ? llam_ql_quantize_q8_1(x, dst, rows_per_call, K, device_id, stream)
                                            : llam_ql_swiglu_quantize(x, src.x2 + (size_t)m * src.ldx, nullptr, dst,
                                                                      rows_per_call, K, device_id, stream);
                        if (!ok)
                            return false;
                    }
                    src = act_source_q8(d_q8_scratch);
                    continue; // groups may form again on the Q8_1 input
                }
                if (!dispatch(fn, projs[i].fmt, projs[i].d_w, projs[i].d_plane, src.q8, projs[i].d_y, nullptr, M,
                              projs[i].N, K, projs[i].ldy, 0, 0, device_id, as_stream(stream)))
                    return false;
                ++i;
            }
            return true;
        }

        bool check_projections(const char *fn, const llam_ql_proj *projs, int num, int M, int K)
        {
            if (num < 0 || num > LLAM_QL_MAX_FUSED)
                return fail(fn, "num=%d outside 0..%d", num, LLAM_QL_MAX_FUSED);
            if (num > 0 && !projs)
                return fail(fn, "null projection table");
            for (int i = 0; i < num; ++i)
            {
                if (!check_matrix(fn, projs[i].fmt, projs[i].d_w, M, projs[i].N, K) ||
                    !check_plane(fn, projs[i].fmt, projs[i].d_plane, projs[i].N, K))
                    return false;
                if (!projs[i].d_y || projs[i].ldy < projs[i].N)
                    return fail(fn, "projection %d: bad output (ldy=%d N=%d)", i, projs[i].ldy, projs[i].N);
            }
            return true;
        }

        bool check_f32(const char *fn, const float *x, int ldx, int K, const void *d_q8_scratch)
        {
            if (!x)
                return fail(fn, "null activations");
            if (ldx < K || (ldx % 4) != 0 || !aligned16(x))
                return fail(fn, "fp32 activations need 16-byte aligned rows (ldx=%d K=%d)", ldx, K);
            if (d_q8_scratch && !aligned4(d_q8_scratch))
                return fail(fn, "d_q8_scratch must be 4-byte aligned");
            return true;
        }
    } // namespace
} // namespace llamql

extern "C" bool llam_ql_gemv_fused(const llam_ql_proj *projs, int num, const void *d_q8,
                                   int M, int K, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_fused";
    if (!check_projections(fn, projs, num, M, K))
        return false;
    if (num == 0)
        return true;
    if (!d_q8 || !aligned4(d_q8))
        return fail(fn, "d_q8 must be a 4-byte aligned device pointer");
    if (!set_device(fn, device_id))
        return false;
    return run_projections(fn, projs, num, act_source_q8(d_q8), M, K, nullptr, device_id, stream);
}

extern "C" bool llam_ql_gemv_f32(uint8_t fmt, const void *d_w, const float *d_x, int ldx, float *d_y,
                                 int M, int N, int K, int ldy, void *d_q8_scratch, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_f32";
    llam_ql_proj p;
    p.d_w = d_w;
    p.d_y = d_y;
    p.N = N;
    p.ldy = ldy;
    p.fmt = fmt;
    p.d_plane = nullptr;
    if (!check_projections(fn, &p, 1, M, K) || !check_f32(fn, d_x, ldx, K, d_q8_scratch))
        return false;
    if (!set_device(fn, device_id))
        return false;
    return run_projections(fn, &p, 1, ActSource{ACT_SRC_F32, nullptr, d_x, nullptr, ldx}, M, K, d_q8_scratch,
                           device_id, stream);
}

// ---- the entry point that brings its own scratch ----------------------------------------
// Q8_1 scratch of llam_ql_gemv_f32_static: LLAM_QL_STATIC_SCRATCH_BYTES of device memory that
// every GPU the library runs on holds from load to exit.  In host code the array's name is
// only a handle for hipGetSymbolAddress; kernels and copies get the address looked up below.
static __device__ __align__(256) uint8_t g_q8_static_scratch[LLAM_QL_STATIC_SCRATCH_BYTES];

namespace llamql
{
    namespace
    {
        // Address of g_q8_static_scratch on the current device (each device has its own copy
        // at its own address), looked up once per device.
        void *static_scratch(const char *fn, int device_id)
        {
            constexpr int MAX_DEVICES = 64;
            static std::atomic<void *> ptr[MAX_DEVICES];
            if (device_id < 0 || device_id >= MAX_DEVICES)
            {
                (void)fail(fn, "device_id %d beyond the %d devices the static scratch is tracked for", device_id,
                           MAX_DEVICES);
                return nullptr;
            }
            void *p = ptr[device_id].load(std::memory_order_acquire);
            if (p)
                return p;
            const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_q8_static_scratch));
            if (e != hipSuccess || !p)
            {
                (void)fail(fn, "hipGetSymbolAddress(scratch) on device %d: %s", device_id, hipGetErrorString(e));
                return nullptr;
            }
            ptr[device_id].store(p, std::memory_order_release); // concurrent first calls find the same address
            return p;
        }
    } // namespace
} // namespace llamql

extern "C" bool llam_ql_gemv_f32_static(uint8_t fmt, const void *d_w, const float *d_x, int ldx, float *d_y,
                                        int M, int N, int K, int ldy, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_f32_static";
    llam_ql_proj p;
    p.d_w = d_w;
    p.d_y = d_y;
    p.N = N;
    p.ldy = ldy;
    p.fmt = fmt;
    p.d_plane = nullptr;
    if (!check_projections(fn, &p, 1, M, K) || !check_f32(fn, d_x, ldx, K, nullptr))
        return false;
    const size_t need = (size_t)M * (size_t)(K / 32) * sizeof(llam_block_q8_1);
    if (need > (size_t)LLAM_QL_STATIC_SCRATCH_BYTES)
        return fail(fn, "M=%d rows of K=%d need %zu bytes of Q8_1 scratch, the built-in buffer holds %d", M, K, need,
                    LLAM_QL_STATIC_SCRATCH_BYTES);
    if (!set_device(fn, device_id))
        return false;
    void *scratch = static_scratch(fn, device_id);
    if (!scratch)
        return false;
    // Every block a call reads from the buffer it has written first: nothing needs clearing.
    return run_projections(fn, &p, 1, ActSource{ACT_SRC_F32, nullptr, d_x, nullptr, ldx}, M, K, scratch, device_id,
                           stream);
}

extern "C" bool llam_ql_gemv_fused_f32(const llam_ql_proj *projs, int num, const float *d_x, int ldx,
                                       int M, int K, void *d_q8_scratch, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_fused_f32";
    if (!check_projections(fn, projs, num, M, K))
        return false;
    if (num == 0)
        return true;
    if (!check_f32(fn, d_x, ldx, K, d_q8_scratch))
        return false;
    if (!set_device(fn, device_id))
        return false;
    return run_projections(fn, projs, num, ActSource{ACT_SRC_F32, nullptr, d_x, nullptr, ldx}, M, K, d_q8_scratch,
                           device_id, stream);
}

extern "C" bool llam_ql_gemv_swiglu_f32(uint8_t fmt, const void *d_w, const void *d_plane, const float *d_gate,
                                        const float *d_up, int ld_gu, float *d_y, int M, int N, int K, int ldy,
                                        void *d_q8_scratch, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_swiglu_f32";
    llam_ql_proj p;
    p.d_w = d_w;
    p.d_y = d_y;
    p.N = N;
    p.ldy = ldy;
    p.fmt = fmt;
    p.d_plane = d_plane;
    if (!check_projections(fn, &p, 1, M, K) || !check_f32(fn, d_gate, ld_gu, K, d_q8_scratch) ||
        !check_f32(fn, d_up, ld_gu, K, nullptr))
        return false;
    if (!set_device(fn, device_id))
        return false;
    return run_projections(fn, &p, 1, ActSource{ACT_SRC_SWIGLU, nullptr, d_gate, d_up, ld_gu}, M, K, d_q8_scratch,
                           device_id, stream);
}

extern "C" bool llam_ql_gemv_accumulate_supported(uint8_t fmt, int M, int N, int K, int device_id)
{
    using namespace llamql;
    if ((fmt != LLAM_FMT_Q4_K && fmt != LLAM_FMT_Q6_K && fmt != LLAM_FMT_IQ3_S) || M < 1 || M > LLAM_QL_MAX_GEMV_M ||
        N < 1 || K < 256 || (K % 256) != 0)
        return false;
    return gemv_accumulate("llam_ql_gemv_accumulate_supported", fmt, nullptr, nullptr, nullptr, M, N, K, N, device_id,
                           nullptr, true);
}

extern "C" bool llam_ql_gemv_accumulate(uint8_t fmt, const void *d_w, const void *d_q8, float *d_y, int M, int N,
                                        int K, int ldy, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_accumulate";
    if (!check_common(fn, fmt, d_w, d_q8, M, N, K))
        return false;
    if (!d_y)
        return fail(fn, "null output");
    if (ldy < N)
        return fail(fn, "ldy=%d smaller than N=%d", ldy, N);
    if (!set_device(fn, device_id))
        return false;
    return gemv_accumulate(fn, fmt, d_w, d_q8, d_y, M, N, K, ldy, device_id, as_stream(stream), false);
}

extern "C" bool llam_ql_gemv_fused_rmsnorm_supported(const llam_ql_proj *projs, int num, int M, int K)
{
    using namespace llamql;
    if (!projs || num < 1 || num > LLAM_QL_MAX_FUSED || K < 256 || (K % 256) != 0)
        return false;
    for (int i = 0; i < num; ++i)
        if (projs[i].N < 1 || !gemv_norm_fusable(projs[i].fmt, M, projs[i].N, K))
            return false;
    return true;
}

extern "C" bool llam_ql_gemv_fused_rmsnorm(const llam_ql_proj *projs, int num, const float *d_x, const float *d_delta,
                                           const float *d_gamma, float eps, float *d_x_out, int M, int K,
                                           int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_fused_rmsnorm";
    if (!check_projections(fn, projs, num, M, K))
        return false;
    if (num == 0)
        return fail(fn, "no projection: the norm runs inside their kernels");
    if (!check_f32(fn, d_x, K, K, nullptr))
        return false;
    if (!d_gamma || !aligned16(d_gamma))
        return fail(fn, "gamma must be a 16-byte aligned device pointer");
    if (d_delta)
    {
        // workgroup 0 writes x + delta while every other workgroup still reads x and delta
        const size_t n = (size_t)M * (size_t)K;
        auto overlaps = [n](const float *a, const float *b) { return a < b + n && b < a + n; };
        if (!aligned16(d_delta) || !d_x_out || !aligned16(d_x_out) || overlaps(d_x_out, d_x) || overlaps(d_x_out, d_delta))
            return fail(fn, "with a delta, x + delta goes to d_x_out: 16-byte aligned, overlapping neither d_x nor d_delta");
    }
    if (!llam_ql_gemv_fused_rmsnorm_supported(projs, num, M, K))
        return fail(fn, "M=%d K=%d: not every projection's kernel can fuse the norm (ask "
                        "llam_ql_gemv_fused_rmsnorm_supported; otherwise norm and projections run as two calls)",
                    M, K);
    if (!set_device(fn, device_id))
        return false;
    ActSource src{ACT_SRC_RMSNORM, nullptr, d_x, d_delta, K};
    src.gamma = d_gamma;
    src.eps = eps;
    src.x_out = d_delta ? d_x_out : nullptr;
    for (int i = 0; i < num;)
    {
        const int took = gemv_group_launch(fn, projs + i, num - i, src, M, K, device_id, as_stream(stream));
        if (took <= 0)
            return took < 0 ? false : fail(fn, "projection %d found no fused launch", i);
        i += took;
    }
    return true;
}

extern "C" bool llam_ql_gemv_block_sums(uint8_t fmt, const void *d_w, const void *d_plane, const void *d_q8,
                                        int32_t *d_sums, int M, int N, int K, int row0,
                                        int nrows, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_block_sums";
    if (!check_common(fn, fmt, d_w, d_q8, M, N, K) || !check_plane(fn, fmt, d_plane, N, K))
        return false;
    if (!d_sums)
        return fail(fn, "null output");
    if (row0 < 0 || nrows < 1 || (long)row0 + nrows > N)
        return fail(fn, "row window [%d,%d) outside [0,%d)", row0, row0 + nrows, N);
    if ((size_t)M * (size_t)nrows * (size_t)(K / 32) * sizeof(int32_t) >= ((size_t)1 << 31))
        return fail(fn, "M=%d x %d rows x %d blocks of sums exceed 2 GiB", M, nrows, K / 32);
    if (!set_device(fn, device_id))
        return false;
    return dispatch(fn, fmt, d_w, d_plane, d_q8, nullptr, d_sums, M, N, K, 0, row0, nrows, device_id, as_stream(stream));
}

extern "C" bool llam_ql_gemv_describe(uint8_t fmt, int M, int N, int K, int has_plane, int device_id,
                                      llam_ql_gemv_plan *out)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemv_describe";
    if (!out)
        return fail(fn, "null output");
    if (fmt != LLAM_FMT_Q4_K && fmt != LLAM_FMT_Q6_K && fmt != LLAM_FMT_IQ3_S)
        return fail(fn, "unsupported weight format id %d", (int)fmt);
    if (M < 1 || M > LLAM_QL_MAX_GEMV_M || N < 1 || K < 1 || (K % 256) != 0)
        return fail(fn, "bad shape (M=%d N=%d K=%d)", M, N, K);
    gemv_describe(fmt, M, N, K, has_plane != 0, device_id, out); // no device call: the unit count falls back to 256
    return true;
}
