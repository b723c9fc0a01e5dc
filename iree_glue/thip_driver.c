// The HAL driver object of "thip": enumerates the one default device and creates it.  Counterpart of
// runtime/driver/torq_driver.c:35-157.  The device it creates is the reference's own synchronous device
// (iree_hal_torq_device_create, runtime/driver/torq_device.h:36-41) over IREE's heap allocator: its executable cache
// (runtime/driver/nop_executable_cache.cc, with the two hunks of README.md) prepares "thip-gfx950" executables, its
// command buffer (runtime/driver/torq_command_buffer.c, one hunk) dispatches them, and its buffers reach the library
// as host pointers, which the library stages.  No CPU executable loaders: a module compiled for this target holds none.
#include "thip_driver.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "thip.h"
#include "torq_device.h"

typedef struct iree_hal_thip_driver_t {
  iree_hal_resource_t resource;
  iree_allocator_t host_allocator;
  int32_t default_ordinal;
  iree_string_view_t identifier;  // storage follows the struct
} iree_hal_thip_driver_t;

static const iree_hal_driver_vtable_t iree_hal_thip_driver_vtable;

static iree_hal_thip_driver_t* iree_hal_thip_driver_cast(iree_hal_driver_t* base) {
  IREE_HAL_ASSERT_TYPE(base, &iree_hal_thip_driver_vtable);
  return (iree_hal_thip_driver_t*)base;
}

iree_status_t iree_hal_thip_driver_create(iree_string_view_t identifier, int32_t default_ordinal, iree_allocator_t host_allocator,
                                          iree_hal_driver_t** out_driver) {
  IREE_ASSERT_ARGUMENT(out_driver);
  *out_driver = NULL;
  iree_hal_thip_driver_t* driver = NULL;
  const iree_host_size_t total = sizeof(*driver) + identifier.size;
  IREE_RETURN_IF_ERROR(iree_allocator_malloc(host_allocator, total, (void**)&driver));
  iree_hal_resource_initialize(&iree_hal_thip_driver_vtable, &driver->resource);
  driver->host_allocator = host_allocator;
  driver->default_ordinal = default_ordinal;
  iree_string_view_append_to_buffer(identifier, &driver->identifier, (char*)driver + sizeof(*driver));
  *out_driver = (iree_hal_driver_t*)driver;
  return iree_ok_status();
}

static void iree_hal_thip_driver_destroy(iree_hal_driver_t* base) {
  iree_hal_thip_driver_t* driver = iree_hal_thip_driver_cast(base);
  iree_allocator_free(driver->host_allocator, driver);
}

static iree_status_t iree_hal_thip_driver_query_available_devices(iree_hal_driver_t* base, iree_allocator_t host_allocator,
                                                                  iree_host_size_t* out_count, iree_hal_device_info_t** out_infos) {
  // one entry: the GPU this driver was created for (other ordinals are reachable through create_device_by_id)
  static const iree_hal_device_info_t infos[1] = {{.device_id = IREE_HAL_DEVICE_ID_DEFAULT, .name = IREE_SVL("gfx950")}};
  *out_count = IREE_ARRAYSIZE(infos);
  return iree_allocator_clone(host_allocator, iree_make_const_byte_span(infos, sizeof(infos)), (void**)out_infos);
}

static iree_status_t iree_hal_thip_driver_dump_device_info(iree_hal_driver_t* base, iree_hal_device_id_t device_id,
                                                           iree_string_builder_t* builder) {
  iree_hal_thip_driver_t* driver = iree_hal_thip_driver_cast(base);
  const int32_t ordinal = device_id == IREE_HAL_DEVICE_ID_DEFAULT ? driver->default_ordinal : (int32_t)device_id;
  thip_device_t* probe = NULL;
  if (thip_device_create(ordinal, &probe) != THIP_OK) {
    return iree_string_builder_append_format(builder, "GPU %d: %s\n", ordinal, thip_status_message());
  }
  char name[64] = {0};
  (void)thip_device_name(probe, name, sizeof(name));
  thip_device_destroy(probe);
  return iree_string_builder_append_format(builder, "GPU %d: %s\n", ordinal, name);
}

static iree_status_t iree_hal_thip_driver_create_device_by_id(iree_hal_driver_t* base, iree_hal_device_id_t device_id,
                                                              iree_host_size_t param_count, const iree_string_pair_t* params,
                                                              iree_allocator_t host_allocator, iree_hal_device_t** out_device) {
  iree_hal_thip_driver_t* driver = iree_hal_thip_driver_cast(base);
  const int32_t ordinal = device_id == IREE_HAL_DEVICE_ID_DEFAULT ? driver->default_ordinal : (int32_t)device_id;
  // the executables of a process share one GPU (thip_native_executable.cc reads THIP_DEVICE_ORDINAL with the first)
  char text[16];
  snprintf(text, sizeof(text), "%d", (int)ordinal);
  setenv("THIP_DEVICE_ORDINAL", text, /*overwrite=*/1);
  iree_hal_torq_device_params_t device_params;
  iree_hal_torq_device_params_initialize(&device_params);
  device_params.is_dmabuf_mode = false;
  iree_hal_allocator_t* device_allocator = NULL;
  IREE_RETURN_IF_ERROR(iree_hal_allocator_create_heap(IREE_SV("local"), host_allocator, host_allocator, &device_allocator));
  iree_status_t status = iree_hal_torq_device_create(driver->identifier, &device_params, /*loader_count=*/0, /*loaders=*/NULL,
                                                     device_allocator, host_allocator, out_device);
  iree_hal_allocator_release(device_allocator);
  return status;
}

static iree_status_t iree_hal_thip_driver_create_device_by_path(iree_hal_driver_t* base, iree_string_view_t driver_name,
                                                                iree_string_view_t device_path, iree_host_size_t param_count,
                                                                const iree_string_pair_t* params, iree_allocator_t host_allocator,
                                                                iree_hal_device_t** out_device) {
  // a path is a GPU ordinal in decimal ("thip://1"); empty: the default device
  iree_hal_device_id_t id = IREE_HAL_DEVICE_ID_DEFAULT;
  if (!iree_string_view_is_empty(device_path)) {
    uint32_t ordinal = 0;
    if (!iree_string_view_atoi_uint32(device_path, &ordinal)) {
      return iree_make_status(IREE_STATUS_NOT_FOUND, "device path '%.*s' is not a GPU ordinal", (int)device_path.size, device_path.data);
    }
    id = (iree_hal_device_id_t)ordinal;
  }
  return iree_hal_thip_driver_create_device_by_id(base, id, param_count, params, host_allocator, out_device);
}

static const iree_hal_driver_vtable_t iree_hal_thip_driver_vtable = {
    .destroy = iree_hal_thip_driver_destroy,
    .query_available_devices = iree_hal_thip_driver_query_available_devices,
    .dump_device_info = iree_hal_thip_driver_dump_device_info,
    .create_device_by_id = iree_hal_thip_driver_create_device_by_id,
    .create_device_by_path = iree_hal_thip_driver_create_device_by_path,
};
