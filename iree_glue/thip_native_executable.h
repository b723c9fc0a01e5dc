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

// The executable format string of a thip descriptor ("thip-gfx950"): what the executable cache's can_prepare_format
// compares with and what thip_infer_format reports.
#define IREE_HAL_THIP_EXECUTABLE_FORMAT "thip-gfx950"

// Same shape as iree_hal_torq_native_executable_create (runtime/driver/native_executable.h:42-46), so that the
// reference's executable cache (runtime/driver/nop_executable_cache.cc:96-114) can call either by format.  `device` is
// the HAL device the cache belongs to; every executable of the process shares one thip_device_t on GPU
// `THIP_DEVICE_ORDINAL` (default 0), created with the first executable and destroyed with the last.
iree_status_t iree_hal_thip_native_executable_create(iree_hal_device_t* device, iree_allocator_t host_allocator,
                                                     const iree_hal_executable_params_t* executable_params,
                                                     iree_hal_executable_t** out_executable);

// Whether a HAL executable is one of this file's (the command buffer's dispatch branches on it).
bool iree_hal_thip_native_executable_isa(iree_hal_executable_t* executable);

// The thip_device_t the executables of this process share; NULL while none exists.  (For an allocator that hands
// out thip_device_alloc memory: it must allocate on this handle.)
thip_device_t* iree_hal_thip_device_handle(void);

// One blocking dispatch.  `binding_is_device[i]` non-zero: binding i is memory of thip_device_alloc and is used in
// place; NULL or zero: it is a host pointer (what the reference's allocators map buffers to) and is staged.
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
