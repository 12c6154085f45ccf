// Error reporting, ABI version and device queries of the C-ABI.
#include "ql_host.h"

#include <cstring>
#include <mutex>
#include <unordered_map>

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

    namespace
    {
        struct BatchPlane
        {
            const uint8_t *plane;
            int N, K;
            uint8_t fmt;
        };
        std::mutex g_plane_mu;
        std::unordered_map<const void *, BatchPlane> g_planes;
    } // namespace

    const uint8_t *batch_plane_of(uint8_t fmt, const void *d_w, int N, int K)
    {
        std::lock_guard<std::mutex> lock(g_plane_mu);
        if (g_planes.empty())
            return nullptr;
        const auto it = g_planes.find(d_w);
        return it != g_planes.end() && it->second.N == N && it->second.K == K && it->second.fmt == fmt ? it->second.plane : nullptr;
    }

    void batch_plane_attach(uint8_t fmt, const void *d_w, const void *d_plane, int N, int K)
    {
        std::lock_guard<std::mutex> lock(g_plane_mu);
        if (d_plane)
            g_planes[d_w] = BatchPlane{static_cast<const uint8_t *>(d_plane), N, K, fmt};
        else
            g_planes.erase(d_w);
    }
} // namespace llamql

extern "C" const char *llam_ql_last_error(void) { return llamql::last_error_text(); }

extern "C" int llam_ql_abi_version(void) { return 1; }
