// Error reporting and version of the C ABI.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "clg_common.h"

namespace {
thread_local char g_error[512] = "";
}

void clg_set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" const char *clg_last_error(void) { return g_error; }
extern "C" int clg_abi_version(void) { return 1; }


// ---- tuning knobs ------------------------------------------------------------------------------
namespace {
const char *const kKnobNames[K_COUNT] = {
#define CLG_KNOB_NAME(name) "CLG_" #name,
    CLG_KNOBS(CLG_KNOB_NAME)
#undef CLG_KNOB_NAME
};
struct KnobTable {
    bool set[K_COUNT];
    char value[K_COUNT][32];
};
KnobTable g_knobs;
std::once_flag g_knobs_once;
void read_knobs()
{
    for (int i = 0; i < K_COUNT; ++i) {
        const char *e = getenv(kKnobNames[i]);
        g_knobs.set[i] = e != nullptr;
        g_knobs.value[i][0] = 0;
        if (e) {
            strncpy(g_knobs.value[i], e, sizeof(g_knobs.value[i]) - 1);
            g_knobs.value[i][sizeof(g_knobs.value[i]) - 1] = 0;
        }
    }
}
}  // namespace

const char *clg_knob(ClgKnob k)
{
    std::call_once(g_knobs_once, read_knobs);
    return g_knobs.set[k] ? g_knobs.value[k] : nullptr;
}

// Not synchronised with launches on other threads: meant for tests and tuning sessions.
extern "C" void clg_reload_knobs(void)
{
    std::call_once(g_knobs_once, read_knobs);
    read_knobs();
}
