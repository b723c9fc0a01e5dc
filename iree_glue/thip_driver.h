// The HAL driver object of "thip".  Counterpart of runtime/driver/torq_driver.h.
#ifndef IREE_GLUE_THIP_DRIVER_H_
#define IREE_GLUE_THIP_DRIVER_H_

#include "iree/base/api.h"
#include "iree/hal/api.h"

#ifdef __cplusplus
extern "C" {
#endif

// One driver instance serves the GPUs of this machine; device ids are GPU ordinals, IREE_HAL_DEVICE_ID_DEFAULT is
// `default_ordinal`.
iree_status_t iree_hal_thip_driver_create(iree_string_view_t identifier, int32_t default_ordinal, iree_allocator_t host_allocator,
                                          iree_hal_driver_t** out_driver);

#ifdef __cplusplus
}
#endif

#endif  // IREE_GLUE_THIP_DRIVER_H_
