// Error reporting, ABI version and device queries of the C-ABI.
#include "ql_host.h"

#include <cstring>
#include <mutex>

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    namespace
    {
        thread_local char g_error[512] = "";
    }

    bool fail(const char *fn, const char *fmt, ...)
    {
        char msg[400];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(msg, sizeof(msg), fmt, ap);
        va_end(ap);
        snprintf(g_error, sizeof(g_error), "[%s] %s", fn, msg);
        fprintf(stderr, "%s\n", g_error);
        return false;
    }

    void clear_error() { g_error[0] = '\0'; }
    const char *last_error_text() { return g_error; }

    int cu_count(int device_id)
    {
        static std::mutex mu;
        static int cached[64];
        std::lock_guard<std::mutex> lock(mu);
        if (device_id < 0 || device_id >= 64)
            return 256;
        if (cached[device_id] == 0)
        {
            int v = 0;
            if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device_id) != hipSuccess || v <= 0)
                v = 256;
            cached[device_id] = v;
        }
        return cached[device_id];
    }
} // namespace llamql

extern "C" const char *llam_ql_last_error(void) { return llamql::last_error_text(); }

extern "C" int llam_ql_abi_version(void) { return 2; }
