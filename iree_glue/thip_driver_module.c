// Registration of the HAL driver "thip" with IREE's driver registry: the counterpart of
// runtime/driver/registration/driver_module.c:95-168 (factory enumerate / try_create for one driver name).
//
// The driver object is thip_driver.c; the device it creates is the reference's own (see there).
#include "iree/base/api.h"
#include "iree/hal/api.h"

#include "thip.h"
#include "thip_driver.h"

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
