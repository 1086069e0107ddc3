// Library-level entry points: version, architecture, status text, device query.
#include <string.h>

#include "dfhip_common.h"

extern "C" int dfhip_version(void) { return 1000; }

extern "C" const char* dfhip_arch(void) { return "gfx950"; }

extern "C" const char* dfhip_status_string(int status) {
  switch (status) {
    case DFHIP_OK: return "ok";
    case DFHIP_ERR_NULL_POINTER: return "null pointer argument";
    case DFHIP_ERR_BAD_SHAPE: return "unsupported shape";
    case DFHIP_ERR_BAD_STRIDE: return "leading dimension smaller than the row length";
    case DFHIP_ERR_BAD_ALIGNMENT: return "pointer or leading dimension not 16-byte aligned";
    case DFHIP_ERR_LAUNCH: return "kernel launch failed";
    case DFHIP_ERR_NO_DEVICE: return "no such HIP device";
    case DFHIP_ERR_BAD_ARGUMENT: return "invalid argument";
    case DFHIP_ERR_TOO_LARGE: return "problem needs more scratch memory than the library holds";
    default: return "unknown status";
  }
}

extern "C" int dfhip_device_info_get(int device, dfhip_device_info* out) {
  if (!out) return DFHIP_ERR_NULL_POINTER;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess) {
    (void)hipGetLastError();
    return DFHIP_ERR_NO_DEVICE;
  }
  out->compute_units = prop.multiProcessorCount;
  out->clock_khz = prop.clockRate;
  out->memory_clock_khz = prop.memoryClockRate;
  out->memory_bus_bits = prop.memoryBusWidth;
  out->lds_bytes_per_block = (int)prop.sharedMemPerBlockOptin;
  out->wavefront_size = prop.warpSize;
  strncpy(out->arch_name, prop.gcnArchName, sizeof(out->arch_name) - 1);
  out->arch_name[sizeof(out->arch_name) - 1] = '\0';
  return DFHIP_OK;
}
