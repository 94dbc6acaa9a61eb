// Host-side helpers shared by the translation units that define C entry points: thread-local error message,
// exception -> status mapping (siglib/cusig/cu_macros.h:27-89), checked sizes (siglib/cpsig/cp_utils.cpp:22-38,91-105).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdio>
#include <mutex>
#include <new>
#include <stdexcept>
#include <string>

namespace sigamd {

extern thread_local char g_last_error[4096];

// Grow-only device buffers, one per (current device, slot), released by cusig_shutdown(); hold g_ws_mutex while a
// buffer is in use (defined in sig_api.hip).  Slots 0-3: signature sweeps; 4-5: sig_join_backprop; 6: word tables of sig_coef; 7, 14, 15: tensor logarithm; 8-11: time-split backward; 12-13: degree-2 backward.
extern std::mutex g_ws_mutex;
void* workspace(int slot, size_t bytes);

// drops the prepared Lyndon tables of every device (defined in sig_log.hip; also called by cusig_shutdown)
void clear_lyndon_tables() noexcept;

inline void clear_last_error() { g_last_error[0] = 0; }
inline void set_last_error(const char* msg) { std::snprintf(g_last_error, sizeof g_last_error, "%s", msg ? msg : ""); }

struct HipFailure : std::runtime_error {
    int code;
    HipFailure(hipError_t e, const char* what_)
        : std::runtime_error(std::string("HIP Error (") + std::to_string(int(e)) + "): " + hipGetErrorString(e) +
                             " [" + what_ + "]"),
          code(int(e)) {}
};

#define SIG_HIP(call)                                              \
    do {                                                           \
        hipError_t e__ = (call);                                   \
        if (e__ != hipSuccess) throw ::sigamd::HipFailure(e__, #call); \
    } while (0)

// Out of device memory, like the reference (siglib/cusig/cu_runtime_utils.h:103-105,212-235): a call whose workspace
// the device cannot hold is retried on halves of its batch; only when a single path does not fit does the call fail,
// as a device error (status 100000 + hipErrorOutOfMemory).  run(first, count) handles `count` batch items from
// `first` on and throws std::bad_alloc when a workspace cannot be had.  A half that failed may already have written
// part of its outputs; the retry overwrites them.
void note_alloc_retry() noexcept;      // counts the splits (defined in sig_api.hip)
template <typename F>
void split_on_bad_alloc(uint64_t batch, const char* who, F&& run)
{
    struct Range {
        uint64_t first, count;
    };
    Range stack[70];        // depth of a binary split of 2^64 items
    int top = 0;
    stack[top++] = Range{0, batch};
    while (top) {
        const Range r = stack[--top];
        try {
            run(r.first, r.count);
        } catch (const std::bad_alloc&) {
            if (r.count <= 1)
                throw HipFailure(hipErrorOutOfMemory, (std::string(who) + ": the workspace of a single batch item does not fit the device").c_str());
            note_alloc_retry();
            const uint64_t half = r.count / 2;
            stack[top++] = Range{r.first + half, r.count - half};
            stack[top++] = Range{r.first, half};
        }
    }
}

// a runtime error that carries its own status code (siglib/shared/errors.h: 5 = prepared cache not found)
struct CodedError : std::runtime_error {
    int code;
    CodedError(int code_, const char* what_) : std::runtime_error(what_), code(code_) {}
};

template <typename F>
int guarded(F&& body) noexcept
{
    clear_last_error();
    try {
        body();
    } catch (const CodedError& e) {
        set_last_error(e.what());
        return e.code;
    } catch (const std::bad_alloc&) {
        set_last_error("Failed to allocate memory");
        return 1;
    } catch (const std::invalid_argument& e) {
        set_last_error(e.what());
        return 2;
    } catch (const std::out_of_range& e) {
        set_last_error(e.what());
        return 3;
    } catch (const HipFailure& e) {
        set_last_error(e.what());
        (void)hipGetLastError();   // do not let a sticky launch error leak into the caller's next call
        return 100000 + e.code;
    } catch (const std::runtime_error& e) {
        set_last_error(e.what());
        return 10;
    } catch (...) {
        set_last_error("Unknown exception");
        return 11;
    }
    return 0;
}

// 0 signals uint64 overflow
inline uint64_t pow_u64(uint64_t base, uint64_t e)
{
    uint64_t r = 1;
    while (e > 0) {
        if (e & 1) {
            if (r != 0 && base > UINT64_MAX / r) return 0;
            r *= base;
        }
        e >>= 1;
        if (e > 0) {
            if (base != 0 && base > UINT64_MAX / base) return 0;
            base *= base;
        }
    }
    return r;
}

inline uint64_t sig_length_u64(uint64_t d, uint64_t degree)
{
    if (d == 0) return 1;
    if (d == 1) return degree + 1;
    const uint64_t p = pow_u64(d, degree + 1);
    return p ? (p - 1) / (d - 1) : 0;
}

inline uint64_t checked_mul(uint64_t a, uint64_t b, const char* what)
{
    if (a != 0 && b > UINT64_MAX / a) throw std::overflow_error(std::string(what) + ": size overflow");
    return a * b;
}

inline unsigned grid_for(uint64_t work, unsigned block = 256)
{
    uint64_t blocks = (work + block - 1) / block;
    if (blocks < 1) blocks = 1;
    if (blocks > 65535u * 16u) blocks = 65535u * 16u;
    return unsigned(blocks);
}

}  // namespace sigamd
