// Device probe and status strings. Stands in for muillm_engine_init
// (csrc/engine.cpp:3-26, csrc/gpu_info.cpp:7-69 in the reference), which records per-GPU
// arch / wave size / SIMD lane count; here a plain struct for the one device in use.
#include <string.h>

#include "common.cuh"

extern "C" int mui_abi_version(void) { return MUI_ABI_VERSION; }

extern "C" const char* mui_status_string(int status) {
  switch (status) {
    case MUI_OK: return "ok";
    case MUI_ERR_INVALID_ARG: return "invalid argument (null pointer, non-positive size or bad enum)";
    case MUI_ERR_UNSUPPORTED: return "shape not supported by the gfx950 kernels";
    case MUI_ERR_LAUNCH: return "kernel launch failed";
    case MUI_ERR_ALIGNMENT: return "pointer or row pitch is not 16-byte aligned";
    case MUI_ERR_DEVICE: return "device query failed";
    default: return "unknown status";
  }
}

extern "C" int mui_device_info(int device, mui_device_info_t* out) {
  if (!out || device < 0) return MUI_ERR_INVALID_ARG;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess) return MUI_ERR_DEVICE;
  memset(out, 0, sizeof(*out));
  out->device = device;
  out->compute_units = prop.multiProcessorCount;
  out->wave_size = prop.warpSize;
  out->simd_lanes = prop.multiProcessorCount * 4 * 16;
  out->lds_bytes_per_block = (int)prop.sharedMemPerBlock;
  out->l2_bytes = prop.l2CacheSize;
  out->clock_khz = prop.clockRate;
  out->hbm_bytes = (uint64_t)prop.totalGlobalMem;
  strncpy(out->arch, prop.gcnArchName, sizeof(out->arch) - 1);
  out->is_gfx950 = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
  return MUI_OK;
}
