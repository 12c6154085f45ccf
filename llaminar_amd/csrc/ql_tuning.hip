// Tuning overrides (for sweeps; production callers never need them).
#include "ql_host.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    namespace
    {
        int g_rows_per_wave = 0;
        int g_unroll = 0;
        int g_mfma_tile_rows = 0;
    }
    int gemv_rows_per_wave_override() { return g_rows_per_wave; }
    int gemv_unroll_override() { return g_unroll; }
    int gemv_mfma_tile_rows_override() { return g_mfma_tile_rows; }
    // Rows of weight per tile of the matrix-unit kernels of batches 5..8 (16..32; anything else:
    // the built-in choice).  Reached from the test-only probe library, not from the C ABI.
    void set_mfma_tile_rows_override(int tile_rows) { g_mfma_tile_rows = tile_rows >= 16 && tile_rows <= 32 ? tile_rows : 0; }
} // namespace llamql

extern "C" void llam_ql_set_gemv_tuning(int rows_per_wave, int unroll)
{
    llamql::g_rows_per_wave = rows_per_wave;
    llamql::g_unroll = unroll;
}
extern "C" void llam_ql_reset_gemv_tuning(void)
{
    llamql::g_rows_per_wave = 0;
    llamql::g_unroll = 0;
}
