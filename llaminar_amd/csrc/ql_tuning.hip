// Tuning overrides (for sweeps; production callers never need them).
#include "ql_host.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    namespace
    {
        int g_rows_per_wave = 0;
        int g_unroll = 0;
    }
    int gemv_rows_per_wave_override() { return g_rows_per_wave; }
    int gemv_unroll_override() { return g_unroll; }
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
