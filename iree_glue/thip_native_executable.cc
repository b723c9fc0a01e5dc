// See thip_native_executable.h.  Follows runtime/driver/native_executable.cc: create :41-108 (copy the program and
// the executable constants, build the executor, initialise it), destroy :110-130, infer_format :151-178, run :180-192.
// The copy, the version / target gates and the per-dispatch lock all live behind the C-ABI; this file only converts
// types and statuses.
#include "thip_native_executable.h"

#include <stdlib.h>
#include <string.h>

#include "iree/base/internal/synchronization.h"

typedef struct iree_hal_thip_native_executable_t {
  iree_hal_resource_t resource;
  iree_allocator_t host_allocator;
  thip_executable_t* executable;
} iree_hal_thip_native_executable_t;

extern const iree_hal_executable_vtable_t iree_hal_thip_native_executable_vtable;

// thip_status_t uses IREE's numbering of the categories it has (include/thip.h).
static iree_status_t iree_hal_thip_status(thip_status_t status) {
  if (status == THIP_OK) return iree_ok_status();
  return iree_make_status((iree_status_code_t)status, "%s", thip_status_message());
}

// The one thip_device_t of the process, counted by the executables that use it.
static iree_slim_mutex_t iree_hal_thip_shared_mutex = IREE_SLIM_MUTEX_INIT;
static thip_device_t* iree_hal_thip_shared_device = NULL;
static int iree_hal_thip_shared_users = 0;

static iree_status_t iree_hal_thip_shared_device_acquire(thip_device_t** out_device) {
  iree_status_t status = iree_ok_status();
  iree_slim_mutex_lock(&iree_hal_thip_shared_mutex);
  if (!iree_hal_thip_shared_device) {
    const char* ordinal = getenv("THIP_DEVICE_ORDINAL");
    status = iree_hal_thip_status(thip_device_create(ordinal ? atoi(ordinal) : 0, &iree_hal_thip_shared_device));
  }
  if (iree_status_is_ok(status)) {
    ++iree_hal_thip_shared_users;
    *out_device = iree_hal_thip_shared_device;
  }
  iree_slim_mutex_unlock(&iree_hal_thip_shared_mutex);
  return status;
}

static void iree_hal_thip_shared_device_release(void) {
  iree_slim_mutex_lock(&iree_hal_thip_shared_mutex);
  if (--iree_hal_thip_shared_users == 0) {
    thip_device_destroy(iree_hal_thip_shared_device);
    iree_hal_thip_shared_device = NULL;
  }
  iree_slim_mutex_unlock(&iree_hal_thip_shared_mutex);
}

thip_device_t* iree_hal_thip_device_handle(void) {
  iree_slim_mutex_lock(&iree_hal_thip_shared_mutex);
  thip_device_t* device = iree_hal_thip_shared_device;
  iree_slim_mutex_unlock(&iree_hal_thip_shared_mutex);
  return device;
}

bool iree_hal_thip_native_executable_isa(iree_hal_executable_t* executable) {
  return iree_hal_resource_is(executable, &iree_hal_thip_native_executable_vtable);
}

static iree_hal_thip_native_executable_t* iree_hal_thip_native_executable_cast(iree_hal_executable_t* base_value) {
  IREE_HAL_ASSERT_TYPE(base_value, &iree_hal_thip_native_executable_vtable);
  return (iree_hal_thip_native_executable_t*)base_value;
}

iree_status_t iree_hal_thip_native_executable_create(iree_hal_device_t* device, iree_allocator_t host_allocator,
                                                     const iree_hal_executable_params_t* executable_params,
                                                     iree_hal_executable_t** out_executable) {
  (void)device;  // buffers reach the dispatch as host pointers whatever device allocated them
  IREE_ASSERT_ARGUMENT(executable_params);
  IREE_ASSERT_ARGUMENT(out_executable);
  *out_executable = NULL;
  IREE_TRACE_ZONE_BEGIN(z0);

  iree_hal_thip_native_executable_t* executable = NULL;
  thip_device_t* thip_device = NULL;
  iree_status_t status = iree_hal_thip_shared_device_acquire(&thip_device);
  if (!iree_status_is_ok(status)) {
    IREE_TRACE_ZONE_END(z0);
    return status;
  }
  status = iree_allocator_malloc(host_allocator, sizeof(*executable), (void**)&executable);
  if (iree_status_is_ok(status)) {
    iree_hal_resource_initialize(&iree_hal_thip_native_executable_vtable, &executable->resource);
    executable->host_allocator = host_allocator;
    executable->executable = NULL;
    // the library copies the blob and the constants: the caller's memory is free again when this returns
    status = iree_hal_thip_status(thip_executable_create(
        thip_device, executable_params->executable_data.data, executable_params->executable_data.data_length,
        executable_params->constants, executable_params->constant_count, &executable->executable));
  }
  if (iree_status_is_ok(status)) {
    *out_executable = (iree_hal_executable_t*)executable;
  } else {
    if (executable) iree_allocator_free(host_allocator, executable);
    iree_hal_thip_shared_device_release();
  }
  IREE_TRACE_ZONE_END(z0);
  return status;
}

static void iree_hal_thip_native_executable_destroy(iree_hal_executable_t* base_executable) {
  iree_hal_thip_native_executable_t* executable = iree_hal_thip_native_executable_cast(base_executable);
  iree_allocator_t host_allocator = executable->host_allocator;
  IREE_TRACE_ZONE_BEGIN(z0);
  thip_executable_destroy(executable->executable);
  iree_allocator_free(host_allocator, executable);
  iree_hal_thip_shared_device_release();
  IREE_TRACE_ZONE_END(z0);
}

iree_status_t iree_hal_thip_native_executable_infer_format(iree_const_byte_span_t executable_data,
                                                           iree_host_size_t executable_format_capacity,
                                                           char* executable_format, iree_host_size_t* out_inferred_size) {
  size_t inferred = 0;
  const thip_status_t status =
      thip_infer_format(executable_data.data, executable_data.data_length, executable_format_capacity, executable_format, &inferred);
  if (status == THIP_INVALID_ARGUMENT) {
    // not one of ours: the executable cache asks every loader in turn
    return iree_make_status(IREE_STATUS_INCOMPATIBLE, "not a thip descriptor: %s", thip_status_message());
  }
  *out_inferred_size = (iree_host_size_t)inferred;
  return iree_hal_thip_status(status);
}

iree_status_t iree_hal_thip_native_executable_run(iree_hal_executable_t* base_executable,
                                                  const iree_hal_executable_dispatch_state_v0_t* dispatch_state,
                                                  const uint8_t* binding_is_device) {
  iree_hal_thip_native_executable_t* executable = iree_hal_thip_native_executable_cast(base_executable);
  // the command buffer has already refused NULL bindings and constants that are no multiple of four bytes
  // (runtime/driver/torq_command_buffer.c:453-494); the library checks the same again against its binding table
  uint8_t flags[64];
  if (dispatch_state->binding_count > IREE_ARRAYSIZE(flags)) {
    return iree_make_status(IREE_STATUS_OUT_OF_RANGE, "%u bindings, at most %u", (unsigned)dispatch_state->binding_count,
                            (unsigned)IREE_ARRAYSIZE(flags));
  }
  for (iree_host_size_t i = 0; i < dispatch_state->binding_count; ++i) {
    flags[i] = (binding_is_device && binding_is_device[i]) ? THIP_BINDING_DEVICE : THIP_BINDING_HOST;
  }
  thip_dispatch_state_t state;
  memset(&state, 0, sizeof(state));
  state.constant_count = dispatch_state->constant_count;
  state.constants = dispatch_state->constants;
  state.binding_count = dispatch_state->binding_count;
  state.binding_ptrs = (void* const*)dispatch_state->binding_ptrs;
  state.binding_lengths = dispatch_state->binding_lengths;
  state.binding_flags = flags;
  IREE_TRACE_ZONE_BEGIN(z0);
  const iree_status_t status = iree_hal_thip_status(thip_executable_run(executable->executable, &state));
  IREE_TRACE_ZONE_END(z0);
  return status;
}

const iree_hal_executable_vtable_t iree_hal_thip_native_executable_vtable = {
    .destroy = iree_hal_thip_native_executable_destroy,
};
