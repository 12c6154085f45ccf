// Host-side plumbing shared by the C-ABI launchers: error text, argument
// checks, device selection.
#pragma once

#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

namespace llamql
{
    // Records "[fn] message" for llam_ql_last_error() and prints it to stderr.
    // Always returns false so launchers can `return fail(...)`.
    bool fail(const char *fn, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
    void clear_error();
    const char *last_error_text();

    inline bool set_device(const char *fn, int device_id)
    {
        int count = 0;
        hipError_t e = hipGetDeviceCount(&count);
        if (e != hipSuccess || count <= 0)
            return fail(fn, "no HIP device available (%s)", hipGetErrorString(e));
        if (device_id < 0 || device_id >= count)
            return fail(fn, "device_id %d out of range [0,%d)", device_id, count);
        e = hipSetDevice(device_id);
        if (e != hipSuccess)
            return fail(fn, "hipSetDevice(%d): %s", device_id, hipGetErrorString(e));
        return true;
    }

    inline bool launched(const char *fn)
    {
        hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return fail(fn, "kernel launch failed: %s", hipGetErrorString(e));
        return true;
    }

    // Dynamic LDS beyond 64 KiB has to be allowed per kernel, once on every device the kernel
    // runs on.  One LdsGrant per launch site remembers the devices that have been served; the
    // flags are atomics because several host threads may launch the same kernel.
    struct LdsGrant
    {
        static constexpr int MAX_DEVICES = 64;
        std::atomic<bool> done[MAX_DEVICES];
    };
    inline hipError_t allow_lds(LdsGrant &g, const void *kernel, size_t bytes)
    {
        int dev = -1;
        if (hipGetDevice(&dev) != hipSuccess)
            dev = -1;
        const bool tracked = dev >= 0 && dev < LdsGrant::MAX_DEVICES;
        if (tracked && g.done[dev].load(std::memory_order_acquire))
            return hipSuccess;
        const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e == hipSuccess && tracked)
            g.done[dev].store(true, std::memory_order_release);
        return e;
    }

    // byte offset of the Q6_K factor plane in a prepared matrix of T super-blocks
    __host__ __device__ inline size_t q6k_factors_offset(size_t T) { return (T * 210 + 15) & ~(size_t)15; }
    // The Q6_K batch plane: the weights of a matrix already requantised to int8, in the order the
    // matrix unit takes them, beside the 16-bit scales of their blocks.  Rows go in groups of
    // four: group g = row / 4 holds, per super-block, eight 128-byte lines (one per 32-column
    // block: the 32 bytes of its four rows one after the other), then, in a second plane, the
    // eight fp16 block scales of each of its rows.
    __host__ __device__ inline size_t q6k_plane_groups(long N) { return (size_t)((N + 3) / 4); }
    __host__ __device__ inline size_t q6k_plane_scales_offset(long N, int nsb) { return q6k_plane_groups(N) * (size_t)nsb * 1024; }
    __host__ __device__ inline size_t q6k_plane_bytes(long N, int nsb) { return q6k_plane_groups(N) * (size_t)nsb * (1024 + 64); }
    // The Q4_K batch plane: the 144 bytes of every super-block regrouped, not changed.  Rows in
    // groups of four; per group and super-block four 128-byte lines (one per 32-byte group of
    // quants: the four rows' 32 bytes in turn), then, in a second plane, the rows' 16-byte heads
    // (d, dmin, scales).
    __host__ __device__ inline size_t q4k_plane_heads_offset(long N, int nsb) { return q6k_plane_groups(N) * (size_t)nsb * 512; }
    __host__ __device__ inline size_t q4k_plane_bytes(long N, int nsb) { return q6k_plane_groups(N) * (size_t)nsb * (512 + 64); }
    inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
    inline bool aligned4(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

    // Number of compute units of the current device (cached per device).
    int cu_count(int device_id);

    inline hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }

    // The activations of a decode GEMV: Q8_1 blocks, or fp32 rows that the kernel quantises
    // itself (plain, or silu(x) * x2 first).
    // ACT_SRC_RMSNORM: the residual rows x (+ delta), RMS-normalised and scaled by gamma.
    constexpr int ACT_SRC_Q8 = 0, ACT_SRC_F32 = 1, ACT_SRC_SWIGLU = 2, ACT_SRC_RMSNORM = 3;
    struct ActSource
    {
        int kind;        // ACT_SRC_*
        const void *q8;  // ACT_SRC_Q8: [M][K/32] blocks
        const float *x;  // ACT_SRC_F32: rows of ldx floats; the gate rows for ACT_SRC_SWIGLU; the
                         // residual rows for ACT_SRC_RMSNORM
        const float *x2; // ACT_SRC_SWIGLU: the up rows; ACT_SRC_RMSNORM: the delta rows to add first, or null
        int ldx;
        const float *gamma = nullptr; // ACT_SRC_RMSNORM: K weights of the norm
        float eps = 0.0f;
        float *x_out = nullptr;       // ACT_SRC_RMSNORM with a delta: where x + delta goes (not x itself)
    };
    inline ActSource act_source_q8(const void *d_q8) { return ActSource{ACT_SRC_Q8, d_q8, nullptr, nullptr, 0}; }
} // namespace llamql
