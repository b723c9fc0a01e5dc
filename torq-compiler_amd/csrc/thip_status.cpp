#include "thip_status.h"

#include <stdarg.h>
#include <stdio.h>

#include "thip_descriptor.h"

namespace thip {

static thread_local char g_message[512] = "";

thip_status_t fail(thip_status_t code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_message, sizeof(g_message), fmt, ap);
    va_end(ap);
    return code;
}

void clearStatus() { g_message[0] = '\0'; }

}  // namespace thip

extern "C" {

const char *thip_status_message(void) { return thip::g_message; }

uint32_t thip_version(void) { return (0u << 16) | 1u; }

uint32_t thip_descriptor_version(void) { return thip::kDescriptorVersion; }

}  // extern "C"
