// Status strings, ABI version and the cached device limits shared by the kernels.
#include "socket_common.h"

const SocketDeviceLimits& socket_device_limits() {
  // One immutable record per process, filled on first use (C++11 guarantees the
  // initialisation is thread-safe).  Falls back to MI355X's figures if the
  // query fails so that size heuristics stay sane.
  static const SocketDeviceLimits lim = [] {
    SocketDeviceLimits l{256, 160 * 1024};
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess) {
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
        l.cu_count = v;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && v > 0)
        l.max_lds_per_block = v;
    }
    return l;
  }();
  return lim;
}

extern "C" int socket_abi_version(void) { return SOCKET_ABI_VERSION; }

extern "C" const char* socket_status_string(int status) {
  switch (status) {
    case SOCKET_OK: return "ok";
    case SOCKET_ERR_NULL: return "a required pointer is NULL";
    case SOCKET_ERR_SHAPE: return "sizes are inconsistent or out of range";
    case SOCKET_ERR_UNSUPPORTED: return "dtype, head dim or table size not supported";
    case SOCKET_ERR_ALIGN: return "pointer or pitch not aligned as required";
    case SOCKET_ERR_WORKSPACE: return "workspace too small";
    case SOCKET_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}

extern "C" int socket_device_query(int* cu_count, int* max_lds_bytes) {
  const SocketDeviceLimits& lim = socket_device_limits();
  if (cu_count) *cu_count = lim.cu_count;
  if (max_lds_bytes) *max_lds_bytes = lim.max_lds_per_block;
  return SOCKET_OK;
}
