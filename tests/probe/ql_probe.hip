// MEASUREMENT AND TEST INFRASTRUCTURE ONLY: built into tests/probe/libql_probe.so, never into
// the product library, and declared in no public header.
//
// Read-only probes: the load streams of the decode GEMV without its arithmetic, for measuring
// what an order of reads is worth on its own (bench.py --workload read-order).  Every probe
// reads the whole buffer once; nothing is written unless the xor of all bytes happens to equal a
// fixed pattern (which keeps the loads alive).
//   llam_probe_read(d_buf, N, K, pattern, rows_per_wave, waves_per_wg, depth, workgroups, d_sink,
//                   device_id, stream): streams the N * (K/256) * 144 bytes of a Q4_K-sized buffer.
//     pattern 0 / 1: the quad-lane kernel's loads (4 lanes per super-block, 3 x 16 bytes per lane
//       and step), N rows shared by ceil(N / rows_per_wave) wavefronts, each with its rows
//       contiguous (0) or dealt round robin (1); depth = steps in flight per wavefront (1, 2, 4).
//     pattern 4 / 5: the walk of 0 / 1 over a buffer in three planes (heads, first and second halves
//       of the lanes' groups), so that no two load instructions touch the same cache line; depth 1..4.
//     pattern 2 / 3: 1 KB per load instruction, `workgroups` workgroups, a region per wavefront
//       (2) or grid-stride (3); depth = loads in flight per lane (3, 6, 9).
//   llam_probe_set_batch_tile_rows(rows): sweep override for the rows of weight per tile (16..32)
//     of the matrix-unit kernels of batches 5..8; any other value restores the built-in choice.
#include "ql_host.h"

#define LLAM_QL_PROBE_ROWS_CONTIGUOUS 0
#define LLAM_QL_PROBE_ROWS_ROUND_ROBIN 1
#define LLAM_QL_PROBE_STREAM_REGION 2
#define LLAM_QL_PROBE_STREAM_GRID_STRIDE 3
#define LLAM_QL_PROBE_PLANES_CONTIGUOUS 4
#define LLAM_QL_PROBE_PLANES_ROUND_ROBIN 5

namespace llamql
{
    void set_mfma_tile_rows_override(int tile_rows); // ql_tuning.hip, not part of the C ABI
}

namespace llamql
{
    typedef int probe_v4i __attribute__((ext_vector_type(4)));

    // The quad-lane kernel's pattern on Q4_K: four lanes per 144-byte super-block, each loading the
    // 16-byte head and its two 16-byte pieces; a wavefront step covers 16 super-blocks of the run
    // formed by the wavefront's rows.  ROUND_ROBIN: wavefront j of tw walks rows j, j + tw, ..;
    // otherwise rows j * rows_per_wave .. of its own.  DEPTH steps are in flight per wavefront.
    // PLANES: the same walk over a buffer laid out in three planes over all T = N * nsb super-blocks,
    // heads [T][16] | first halves of the lanes' groups [T][64] | second halves [T][64]: every load
    // instruction of a wavefront then reads whole runs of bytes nobody else asks for.
    template <bool ROUND_ROBIN, int DEPTH, bool PLANES = false>
    __global__ void __launch_bounds__(1024)
        read_probe_rows_kernel(const uint8_t *p, int N, int nsb, int rows_per_wave, int *sink)
    {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
        const int grp = lane >> 2, l = lane & 3;
        const long j = (long)blockIdx.x * nw + wave;
        const long tw = ((long)N + rows_per_wave - 1) / rows_per_wave;
        long nrows = 0;
        if (j < tw)
        {
            if (ROUND_ROBIN)
                nrows = (N - 1 - j) / tw + 1;
            else
                nrows = j * rows_per_wave + rows_per_wave <= N ? rows_per_wave : N - j * rows_per_wave;
        }
        const int total = (int)nrows * nsb;
        const int nsteps = (total + 15) / 16;
        probe_v4i acc = {0, 0, 0, 0};
        for (int s0 = 0; s0 < nsteps; s0 += DEPTH)
        {
            probe_v4i v[DEPTH][3];
#pragma unroll
            for (int u = 0; u < DEPTH; ++u)
            {
                int s = (s0 + u) * 16 + grp;
                if (s >= total)
                    s = total - 1;
                const int lr = s / nsb, sbr = s - lr * nsb;
                const long row = ROUND_ROBIN ? lr * tw + j : j * rows_per_wave + lr;
                if (PLANES)
                {
                    const size_t T = (size_t)N * nsb, t = (size_t)row * nsb + sbr;
                    v[u][0] = *reinterpret_cast<const probe_v4i *>(p + t * 16);
                    v[u][1] = *reinterpret_cast<const probe_v4i *>(p + T * 16 + t * 64 + 16 * l);
                    v[u][2] = *reinterpret_cast<const probe_v4i *>(p + T * 80 + t * 64 + 16 * l);
                }
                else
                {
                    const uint8_t *sb = p + ((size_t)row * nsb + sbr) * 144;
                    v[u][0] = *reinterpret_cast<const probe_v4i *>(sb);
                    v[u][1] = *reinterpret_cast<const probe_v4i *>(sb + 16 + 32 * l);
                    v[u][2] = *reinterpret_cast<const probe_v4i *>(sb + 32 + 32 * l);
                }
            }
#pragma unroll
            for (int u = 0; u < DEPTH; ++u)
                acc ^= v[u][0] ^ v[u][1] ^ v[u][2];
        }
        if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678)
            sink[0] = 1;
    }

    // A plain stream: every load instruction of a wavefront reads 1 KB.  GRID_STRIDE: wavefront
    // j reads chunks j, j + all wavefronts, ..; otherwise a contiguous region of its own.
    template <bool GRID_STRIDE, int DEPTH>
    __global__ void __launch_bounds__(1024) read_probe_stream_kernel(const uint8_t *p, size_t chunks, int *sink)
    {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
        const size_t j = (size_t)blockIdx.x * nw + wave, tw = (size_t)gridDim.x * nw;
        const size_t per_wave = (chunks + tw - 1) / tw;
        probe_v4i acc = {0, 0, 0, 0};
        for (size_t i0 = 0; i0 < per_wave; i0 += DEPTH)
        {
            probe_v4i v[DEPTH];
#pragma unroll
            for (int u = 0; u < DEPTH; ++u)
            {
                size_t c = GRID_STRIDE ? j + (i0 + u) * tw : j * per_wave + i0 + u;
                if (i0 + u >= per_wave || c >= chunks)
                    c = chunks - 1;
                v[u] = *reinterpret_cast<const probe_v4i *>(p + c * 1024 + lane * 16);
            }
#pragma unroll
            for (int u = 0; u < DEPTH; ++u)
                acc ^= v[u];
        }
        if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678)
            sink[0] = 1;
    }

    template <bool A, bool PLANES = false>
    void launch_rows(int depth, dim3 grid, dim3 block, hipStream_t st, const uint8_t *p, int N, int nsb, int rpw, int *sink)
    {
        switch (depth)
        {
        case 1: hipLaunchKernelGGL((read_probe_rows_kernel<A, 1, PLANES>), grid, block, 0, st, p, N, nsb, rpw, sink); break;
        case 2: hipLaunchKernelGGL((read_probe_rows_kernel<A, 2, PLANES>), grid, block, 0, st, p, N, nsb, rpw, sink); break;
        case 3: hipLaunchKernelGGL((read_probe_rows_kernel<A, 3, PLANES>), grid, block, 0, st, p, N, nsb, rpw, sink); break;
        default: hipLaunchKernelGGL((read_probe_rows_kernel<A, 4, PLANES>), grid, block, 0, st, p, N, nsb, rpw, sink); break;
        }
    }

    template <bool A>
    void launch_stream(int depth, dim3 grid, dim3 block, hipStream_t st, const uint8_t *p, size_t chunks, int *sink)
    {
        switch (depth)
        {
        case 3: hipLaunchKernelGGL((read_probe_stream_kernel<A, 3>), grid, block, 0, st, p, chunks, sink); break;
        case 6: hipLaunchKernelGGL((read_probe_stream_kernel<A, 6>), grid, block, 0, st, p, chunks, sink); break;
        default: hipLaunchKernelGGL((read_probe_stream_kernel<A, 9>), grid, block, 0, st, p, chunks, sink); break;
        }
    }
} // namespace llamql

using namespace llamql;

extern "C" bool llam_probe_read(const void *d_buf, int N, int K, int pattern, int rows_per_wave,
                                int waves_per_wg, int depth, int workgroups, int *d_sink, int device_id,
                                void *stream)
{
    const char *fn = "llam_probe_read";
    clear_error();
    if (!d_buf || !d_sink)
        return fail(fn, "null buffer");
    if (N < 1 || K < 4096 || K % 256 != 0)
        return fail(fn, "N=%d K=%d: rows of at least 16 super-blocks of 256 columns", N, K);
    if (waves_per_wg < 1 || waves_per_wg > 16)
        return fail(fn, "waves_per_wg=%d out of range 1..16", waves_per_wg);
    if (!set_device(fn, device_id))
        return false;
    const int nsb = K / 256;
    hipStream_t st = as_stream(stream);
    const uint8_t *p = static_cast<const uint8_t *>(d_buf);
    const dim3 block((unsigned)waves_per_wg * 64);
    if (pattern == LLAM_QL_PROBE_ROWS_CONTIGUOUS || pattern == LLAM_QL_PROBE_ROWS_ROUND_ROBIN ||
        pattern == LLAM_QL_PROBE_PLANES_CONTIGUOUS || pattern == LLAM_QL_PROBE_PLANES_ROUND_ROBIN)
    {
        if (rows_per_wave < 1 || depth < 1 || depth > 4)
            return fail(fn, "rows_per_wave=%d depth=%d (depth 1..4)", rows_per_wave, depth);
        if ((long)rows_per_wave * nsb > 0x7FFFFFF)
            return fail(fn, "run too long");
        const long tw = ((long)N + rows_per_wave - 1) / rows_per_wave;
        const dim3 grid((unsigned)((tw + waves_per_wg - 1) / waves_per_wg));
        if (pattern == LLAM_QL_PROBE_ROWS_ROUND_ROBIN)
            launch_rows<true>(depth, grid, block, st, p, N, nsb, rows_per_wave, d_sink);
        else if (pattern == LLAM_QL_PROBE_ROWS_CONTIGUOUS)
            launch_rows<false>(depth, grid, block, st, p, N, nsb, rows_per_wave, d_sink);
        else if (pattern == LLAM_QL_PROBE_PLANES_ROUND_ROBIN)
            launch_rows<true, true>(depth, grid, block, st, p, N, nsb, rows_per_wave, d_sink);
        else
            launch_rows<false, true>(depth, grid, block, st, p, N, nsb, rows_per_wave, d_sink);
        return launched(fn);
    }
    if (pattern == LLAM_QL_PROBE_STREAM_REGION || pattern == LLAM_QL_PROBE_STREAM_GRID_STRIDE)
    {
        if (workgroups < 1 || (depth != 3 && depth != 6 && depth != 9))
            return fail(fn, "workgroups=%d depth=%d (depth 3, 6 or 9)", workgroups, depth);
        const size_t chunks = (size_t)N * nsb * 144 / 1024;
        if (chunks < 1)
            return fail(fn, "buffer shorter than one chunk");
        if (pattern == LLAM_QL_PROBE_STREAM_GRID_STRIDE)
            launch_stream<true>(depth, dim3((unsigned)workgroups), block, st, p, chunks, d_sink);
        else
            launch_stream<false>(depth, dim3((unsigned)workgroups), block, st, p, chunks, d_sink);
        return launched(fn);
    }
    return fail(fn, "unknown pattern %d", pattern);
}

extern "C" void llam_probe_set_batch_tile_rows(int tile_rows) { llamql::set_mfma_tile_rows_override(tile_rows); }
