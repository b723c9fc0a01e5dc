// Host-only validation of dispatch descriptors (no HIP calls).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "thip_descriptor.h"
#include "thip_status.h"

namespace thip {

// The tables of a descriptor blob that passed validateDescriptor.
struct DescriptorView {
    const uint8_t *blob;
    DescHeader header;
    const DescOp *ops;
    const DescBinding *bindings;
    const DescTemp *temps;
    const DescConst *consts;
};

// Header, table extents, every operand reference inside its buffer.  Magic / version / arch mismatches are
// THIP_UNAVAILABLE (the reference's runtime_version and hw-id gates), malformed contents THIP_INVALID_ARGUMENT.
thip_status_t validateDescriptor(const uint8_t *blob, size_t size, DescHeader *out);
// That kernel record i stays inside the buffers it names (its k-tables included).
thip_status_t checkOpFootprint(const DescriptorView *view, uint32_t i);
// Both, over every record.
thip_status_t validateWhole(const uint8_t *blob, size_t size, DescHeader *out);

}  // namespace thip
