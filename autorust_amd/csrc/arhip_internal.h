// Internal declarations shared by the translation units of libarhip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/arhip.h"

// A loaded code object, or several of them loaded from one image (a container: see arhip_module_load)
struct arhip_module_entry {
    std::vector<hipModule_t> mods;
    std::vector<std::vector<char>> images;  // private copies, alive as long as the modules are loaded
    std::unordered_map<std::string, hipFunction_t> fns;
};

struct arhip_device {
    int ordinal = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;  // per-call timing (`wait`)
    hipEvent_t tm0 = nullptr, tm1 = nullptr;  // arhip_timer_start/stop
    std::string arch;
    int cus = 0;
    std::unordered_map<uint64_t, arhip_module_entry *> modules;  // by content hash
    // per-launch event pairs while kernel profiling is on (arhip_kprof_*)
    struct prof_entry { int kernel; hipEvent_t e0, e1; };
    bool prof = false;
    std::vector<prof_entry> prof_log;
    std::vector<hipEvent_t> prof_pool;
    bool capturing = false;  // between arhip_graph_begin and arhip_graph_end
    int attn_waves = 0;      // ARHIP_ATTN_WAVES at open (0: choose by shape)
};

// Records a message for arhip_last_error() and returns `code`.
int arhip_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define ARHIP_HIP(call)                                                                      \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess) {                                                              \
            (void)hipGetLastError(); /* do not let it surface in a later, unrelated call */  \
            return arhip_fail(ARHIP_EHIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                              __FILE__, __LINE__);                                           \
        }                                                                                    \
    } while (0)

#define ARHIP_REQUIRE(cond, ...)                                  \
    do {                                                          \
        if (!(cond)) return arhip_fail(ARHIP_EINVAL, __VA_ARGS__); \
    } while (0)

// Brackets a launch with events when the caller asked to wait.
struct arhip_call_timer {
    arhip_device *dev;
    int wait;
    double *secs;
    int kernel = -1;          // ARHIP_K_* for the profile log, -1: not logged
    hipEvent_t p0 = nullptr;  // profile events of this launch
    hipEvent_t p1 = nullptr;
    int begin();
    int end();
};

void arhip_note_selected(int kernel);

// Resolves the device address of the built-in Sage scratch array for the current device.
int arhip_static_scratch_setup(int ordinal);

static inline bool arhip_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
