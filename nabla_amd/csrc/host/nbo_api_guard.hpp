// What every extern "C" entry point is wrapped in: one process-wide lock, and the mapping of
// internal errors to status codes.
#ifndef NBO_API_GUARD_HPP
#define NBO_API_GUARD_HPP

#include <mutex>
#include <new>

#include "nbo_host.hpp"

namespace nbo {

// The runtime's stream, staging buffer and reduction scratch are shared by every
// handle, so entry points run one at a time; the device work they enqueue is ordered
// by the one stream.
std::recursive_mutex &api_mutex();

// Runs `body`, mapping internal errors to status codes; nothing escapes the C ABI.
template <typename F> int guarded(F &&body)
{
    std::lock_guard<std::recursive_mutex> lock(api_mutex());
    try {
        body();
        return NBO_OK;
    } catch (const Error &e) {
        set_last_error(e.msg);
        return e.status;
    } catch (const std::bad_alloc &) {
        set_last_error("host allocation failed");
        return NBO_ERR_ARG;
    } catch (...) {
        set_last_error("unexpected internal error");
        return NBO_ERR_ARG;
    }
}

inline void require(bool cond, int status, const char *msg)
{
    if (!cond) fail(status, msg);
}

} // namespace nbo

#endif
