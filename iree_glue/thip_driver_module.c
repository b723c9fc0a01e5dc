// Registration of the HAL driver "thip" with IREE's driver registry: the counterpart of
// runtime/driver/registration/driver_module.c:95-168 (factory enumerate / try_create for one driver name).
//
// The driver and device objects themselves are the reference's (runtime/driver/torq_driver.c, torq_device.c) with
// three substitutions, all of them calls into include/thip.h:
//   - the device owns one thip_device_t (thip_device_create(ordinal) at creation, thip_device_destroy at the end);
//   - its allocator hands out device-local buffers from thip_device_alloc / thip_device_free and moves data with
//     thip_device_h2d / thip_device_d2h (the roles of TorqHw::allocateDeviceBuffer / writeXram / readXram,
//     runtime/torq_hw/inc/TorqHw.h:96-121); host-visible buffers stay plain host memory and are staged by the library;
//   - its command buffer's dispatch (runtime/driver/torq_command_buffer.c:390-512) builds the dispatch state as
//     before and calls iree_hal_thip_native_executable_run, passing for every binding whether its buffer came from
//     thip_device_alloc.
#include "iree/base/api.h"
#include "iree/hal/api.h"

#include "thip.h"
#include "thip_driver.h"
#include "thip_native_executable.h"

static iree_status_t iree_hal_thip_driver_factory_enumerate(void* self, iree_host_size_t* out_driver_info_count,
                                                            const iree_hal_driver_info_t** out_driver_infos) {
  static const iree_hal_driver_info_t driver_info = {
      .driver_name = IREE_SVL("thip"),
      .full_name = IREE_SVL("Quantized TorqHL operator path on AMD Instinct MI355X (gfx950)"),
  };
  *out_driver_info_count = 1;
  *out_driver_infos = &driver_info;
  return iree_ok_status();
}

static iree_status_t iree_hal_thip_driver_factory_try_create(void* self, iree_string_view_t driver_name,
                                                             iree_allocator_t host_allocator, iree_hal_driver_t** out_driver) {
  if (!iree_string_view_equal(driver_name, IREE_SV("thip"))) {
    return iree_make_status(IREE_STATUS_UNAVAILABLE, "no driver '%.*s' is provided by this factory", (int)driver_name.size,
                            driver_name.data);
  }
  // Is there a gfx950 at all?  The library answers UNAVAILABLE without one, which is what the registry expects from
  // a driver that cannot run here.
  thip_device_t* probe = NULL;
  const thip_status_t status = thip_device_create(0, &probe);
  if (status != THIP_OK) return iree_make_status((iree_status_code_t)status, "%s", thip_status_message());
  thip_device_destroy(probe);
  return iree_hal_thip_driver_create(driver_name, /*device_ordinal=*/0, host_allocator, out_driver);
}

IREE_API_EXPORT iree_status_t iree_hal_thip_driver_module_register(iree_hal_driver_registry_t* registry) {
  static const iree_hal_driver_factory_t factory = {
      .self = NULL,
      .enumerate = iree_hal_thip_driver_factory_enumerate,
      .try_create = iree_hal_thip_driver_factory_try_create,
  };
  return iree_hal_driver_registry_register_factory(registry, &factory);
}
