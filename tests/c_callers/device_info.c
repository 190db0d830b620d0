/* Device and memory API walk-through: every odla_GetDeviceInfo item must answer
 * ODLA_SUCCESS on the default device [ref: tests/ODLA/device_test.cc:63-89], and
 * host / device memory from the library round-trips data through
 * odla_CopyMemory [ref: ODLA/include/ODLA/odla_memory.h:47-87]. */
#include <odla_hip.h>
#include <stdio.h>
#include <string.h>

#define ITEM(x) {x, #x}

int main(void) {
  odla_device dev = NULL;
  if (odla_AllocateDevice(NULL, ODLA_DEVICE_DEFAULT, 0, &dev) != ODLA_SUCCESS || dev == NULL) {
    printf("odla_AllocateDevice failed\n");
    return 1;
  }
  const struct { odla_device_info item; const char* name; } items[] = {
      ITEM(ODLA_DEVICE_INFO_ODLA_LIB_VERSION), ITEM(ODLA_DEVICE_INFO_DEV_COUNT),
      ITEM(ODLA_DEVICE_INFO_DEV_INDEX),        ITEM(ODLA_DEVICE_INFO_DEV_TYPE),
      ITEM(ODLA_DEVICE_INFO_DEV_UUID),         ITEM(ODLA_DEVICE_INFO_PROCESSOR_UTIL),
      ITEM(ODLA_DEVICE_INFO_MEMORY_UTIL),      ITEM(ODLA_DEVICE_INFO_TOTAL_MEMORY),
      ITEM(ODLA_DEVICE_INFO_USED_MEMORY),      ITEM(ODLA_DEVICE_INFO_POWER_USAGE),
      ITEM(ODLA_DEVICE_INFO_POWER_LIMIT),      ITEM(ODLA_DEVICE_INFO_DRIVER_VERSION),
      ITEM(ODLA_DEVICE_INFO_SDK_VERSION)};
  for (unsigned i = 0; i < sizeof(items) / sizeof(items[0]); ++i) {
    odla_scalar_value val;
    memset(&val, 0, sizeof(val));
    if (odla_GetDeviceInfo(dev, items[i].item, &val) != ODLA_SUCCESS) {
      printf("Failed to get %s\n", items[i].name);
      return 1;
    }
    printf("%s: ", items[i].name);
    switch (val.data_type) {
      case ODLA_INT32: printf("%d\n", val.val_int32); break;
      case ODLA_INT64: printf("%lld\n", (long long)val.val_int64); break;
      case ODLA_FLOAT32: printf("%f\n", val.val_fp32); break;
      case ODLA_STRING: printf("%s\n", items[i].item == ODLA_DEVICE_INFO_DEV_UUID ? "(16 bytes)" : val.val_str); break;
      default: printf("--\n");
    }
    if (items[i].item == ODLA_DEVICE_INFO_DEV_COUNT && val.val_int32 < 1) return 1;
    if (items[i].item == ODLA_DEVICE_INFO_TOTAL_MEMORY && val.val_int64 <= 0) return 1;
  }
  if (odla_SetCurrentDevice(dev) != ODLA_SUCCESS) return 1;

  /* host -> device -> device -> host */
  enum { N = 1 << 16 };
  odla_void *h0 = NULL, *h1 = NULL, *d0 = NULL, *d1 = NULL;
  if (odla_AllocateHostMemory(&h0, N) != ODLA_SUCCESS || odla_AllocateHostMemory(&h1, N) != ODLA_SUCCESS ||
      odla_AllocateDeviceMemory(&d0, N) != ODLA_SUCCESS || odla_AllocateDeviceMemory(&d1, N) != ODLA_SUCCESS) {
    printf("allocation failed\n");
    return 1;
  }
  for (int i = 0; i < N; ++i) ((unsigned char*)h0)[i] = (unsigned char)(i * 7 + 3);
  memset(h1, 0, N);
  if (odla_CopyMemory(d0, h0, N, ODLA_MEMCPY_H2D) != ODLA_SUCCESS ||
      odla_CopyMemory(d1, d0, N, ODLA_MEMCPY_D2D) != ODLA_SUCCESS ||
      odla_CopyMemory(h1, d1, N, ODLA_MEMCPY_D2H) != ODLA_SUCCESS) {
    printf("copy failed\n");
    return 1;
  }
  if (memcmp(h0, h1, N) != 0) {
    printf("round trip mismatch\n");
    return 1;
  }
  if (odla_FreeHostMemory(h0) != ODLA_SUCCESS || odla_FreeHostMemory(h1) != ODLA_SUCCESS ||
      odla_FreeDeviceMemory(d0) != ODLA_SUCCESS || odla_FreeDeviceMemory(d1) != ODLA_SUCCESS)
    return 1;
  if (odla_AllocateHostMemory(NULL, 16) == ODLA_SUCCESS) return 1; /* a null result pointer is refused */
  if (odla_DestroyDevice(dev) != ODLA_SUCCESS) return 1;
  printf("memory round trip ok\n");
  return 0;
}
