// A range of device addresses that keeps its place while the memory behind it is given back and taken again.
//
// The engine state of the boundary-form GatedDeltaNet layers sleeps with the engine: the reference carves each layer's
// state out of one tagged allocation of the engine's virtual-memory allocator, which sleep discards without a host copy
// and wake maps again at the same address, so that captured decode graphs -- which hold addresses -- stay valid
// (ops/gdn/gdn_cpr_sleep.py:45-124, 217-282). This is the same thing on the HIP virtual-memory calls: one address
// reservation per arena for the life of the process, physical memory created and mapped on create / restore, unmapped
// and released on release. Set-up calls: they allocate, and release synchronises the device (nothing may still be
// using the memory that goes away). Touching the range while it is released is a memory fault: the caller keeps
// everything that could (tensors, graph replays) away from it until restore has returned.
#include "ix_common.h"
#include "../../include/isoexec_hip.h"

struct IxArena {
  void* base;
  size_t bytes;  // a multiple of the allocation granularity
  int device;
  bool mapped;
  hipMemGenericAllocationHandle_t handle;
};

static hipMemAllocationProp ix_arena_prop(int device) {
  hipMemAllocationProp prop = {};
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.location.id = device;
  return prop;
}

static int ix_arena_map(IxArena* a) {
  const hipMemAllocationProp prop = ix_arena_prop(a->device);
  if (hipMemCreate(&a->handle, a->bytes, &prop, 0) != hipSuccess) return IX_ERR_SIZE;  // no memory of that size
  if (hipMemMap(a->base, a->bytes, 0, a->handle, 0) != hipSuccess) {
    hipMemRelease(a->handle);
    return IX_ERR_LAUNCH;
  }
  hipMemAccessDesc access = {};
  access.location = prop.location;
  access.flags = hipMemAccessFlagsProtReadWrite;
  if (hipMemSetAccess(a->base, a->bytes, &access, 1) != hipSuccess) {
    hipMemUnmap(a->base, a->bytes);
    hipMemRelease(a->handle);
    return IX_ERR_LAUNCH;
  }
  a->mapped = true;
  return IX_OK;
}

extern "C" int ix_arena_create(size_t bytes, void** arena_out, void* stream) {
  if (!arena_out || bytes == 0) return IX_ERR_ARG;
  *arena_out = nullptr;
  int device = 0, supported = 0;
  if (hipGetDevice(&device) != hipSuccess) return IX_ERR_LAUNCH;
  if (hipDeviceGetAttribute(&supported, hipDeviceAttributeVirtualMemoryManagementSupported, device) != hipSuccess ||
      !supported)
    return IX_DECLINED;
  const hipMemAllocationProp prop = ix_arena_prop(device);
  size_t gran = 0;
  if (hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityMinimum) != hipSuccess || gran == 0)
    return IX_DECLINED;
  if (gran < 256) gran = 256;
  IxArena* a = new IxArena();
  a->bytes = (bytes + gran - 1) / gran * gran;
  a->device = device;
  a->mapped = false;
  a->base = nullptr;
  if (hipMemAddressReserve(&a->base, a->bytes, 0, nullptr, 0) != hipSuccess || !a->base) {
    delete a;
    return IX_ERR_SIZE;
  }
  const int rc = ix_arena_map(a);
  if (rc != IX_OK) {
    hipMemAddressFree(a->base, a->bytes);
    delete a;
    return rc;
  }
  if (hipMemsetAsync(a->base, 0, a->bytes, (hipStream_t)stream) != hipSuccess) {
    hipMemUnmap(a->base, a->bytes);
    hipMemRelease(a->handle);
    hipMemAddressFree(a->base, a->bytes);
    delete a;
    return IX_ERR_LAUNCH;
  }
  *arena_out = a;
  return IX_OK;
}

extern "C" void* ix_arena_base(const void* arena) { return arena ? static_cast<const IxArena*>(arena)->base : nullptr; }
extern "C" size_t ix_arena_bytes(const void* arena) { return arena ? static_cast<const IxArena*>(arena)->bytes : 0; }
extern "C" int ix_arena_is_mapped(const void* arena) { return arena && static_cast<const IxArena*>(arena)->mapped ? 1 : 0; }

extern "C" int ix_arena_release_memory(void* arena) {
  if (!arena) return IX_ERR_ARG;
  IxArena* a = static_cast<IxArena*>(arena);
  if (!a->mapped) return IX_OK;
  int current = 0;
  if (hipGetDevice(&current) != hipSuccess || current != a->device) return IX_ERR_ARG;
  if (hipDeviceSynchronize() != hipSuccess) return IX_ERR_LAUNCH;  // nothing in flight may still address the range
  if (hipMemUnmap(a->base, a->bytes) != hipSuccess) return IX_ERR_LAUNCH;
  a->mapped = false;
  if (hipMemRelease(a->handle) != hipSuccess) return IX_ERR_LAUNCH;
  return IX_OK;
}

extern "C" int ix_arena_restore_memory(void* arena, void* stream) {
  if (!arena) return IX_ERR_ARG;
  IxArena* a = static_cast<IxArena*>(arena);
  if (a->mapped) return IX_OK;
  int current = 0;
  if (hipGetDevice(&current) != hipSuccess || current != a->device) return IX_ERR_ARG;
  const int rc = ix_arena_map(a);
  if (rc != IX_OK) return rc;
  if (hipMemsetAsync(a->base, 0, a->bytes, (hipStream_t)stream) != hipSuccess) return IX_ERR_LAUNCH;
  return IX_OK;
}

extern "C" int ix_arena_destroy(void* arena) {
  if (!arena) return IX_ERR_ARG;
  IxArena* a = static_cast<IxArena*>(arena);
  const int rc = ix_arena_release_memory(a);
  if (rc != IX_OK) return rc;
  if (hipMemAddressFree(a->base, a->bytes) != hipSuccess) return IX_ERR_LAUNCH;
  delete a;
  return IX_OK;
}
