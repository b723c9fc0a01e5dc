// HAL executable of the "thip" driver: a thip_executable_t behind IREE's executable interface.  Counterpart of
// runtime/driver/native_executable.h:24-58.
#ifndef IREE_GLUE_THIP_NATIVE_EXECUTABLE_H_
#define IREE_GLUE_THIP_NATIVE_EXECUTABLE_H_

#include "iree/base/api.h"
#include "iree/hal/api.h"
#include "iree/hal/local/executable_library.h"

#include "thip.h"

#ifdef __cplusplus
extern "C" {
#endif

// `thip_device` is the one thip_device_t the HAL device owns.
iree_status_t iree_hal_thip_native_executable_create(thip_device_t* thip_device, iree_allocator_t host_allocator,
                                                     const iree_hal_executable_params_t* executable_params,
                                                     iree_hal_executable_t** out_executable);

// One blocking dispatch.  `binding_is_device[i]` non-zero: binding i is memory of thip_device_alloc (a device-local HAL
// buffer of this driver) and is used in place; otherwise it is a host pointer and is staged.
iree_status_t iree_hal_thip_native_executable_run(iree_hal_executable_t* executable,
                                                  const iree_hal_executable_dispatch_state_v0_t* dispatch_state,
                                                  const uint8_t* binding_is_device);

iree_status_t iree_hal_thip_native_executable_infer_format(iree_const_byte_span_t executable_data,
                                                           iree_host_size_t executable_format_capacity,
                                                           char* executable_format, iree_host_size_t* out_inferred_size);

#ifdef __cplusplus
}
#endif

#endif  // IREE_GLUE_THIP_NATIVE_EXECUTABLE_H_
