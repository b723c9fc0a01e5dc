// The HAL device of the "thip" driver: what thip_driver.c, thip_native_executable.cc and the dispatch path need from it.
// Counterpart of runtime/driver/torq_device.h:20-40.  The device object itself is NOT in this directory yet (see
// README.md): it is the reference's synchronous device (runtime/driver/torq_device.c) owning one thip_device_t.
#ifndef IREE_GLUE_THIP_DEVICE_H_
#define IREE_GLUE_THIP_DEVICE_H_

#include "iree/base/api.h"
#include "iree/hal/api.h"

#include "thip.h"

#ifdef __cplusplus
extern "C" {
#endif

// Creates the device for GPU `device_ordinal`: thip_device_create(device_ordinal) at creation, thip_device_destroy when
// the last reference goes.  UNAVAILABLE without a gfx950 GPU or without libthip.so's kernels (the library's own status).
iree_status_t iree_hal_thip_device_create(iree_string_view_t identifier, int32_t device_ordinal, iree_allocator_t host_allocator,
                                          iree_hal_device_t** out_device);

// The thip_device_t a HAL device of this driver owns (borrowed; valid while the device lives).
thip_device_t* iree_hal_thip_device_handle(iree_hal_device_t* device);

#ifdef __cplusplus
}
#endif

#endif  // IREE_GLUE_THIP_DEVICE_H_
