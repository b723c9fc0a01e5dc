// Status plumbing shared by the emitter and the driver: a thread-local message
// behind thip_status_message() and a printf-style helper that sets it.
#pragma once

#include "../../include/thip.h"

namespace thip {

// Records the message for this thread and returns `code`.
thip_status_t fail(thip_status_t code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clearStatus();

}  // namespace thip
