// Functions shared by the translation units of libhc_amd_runtime.so; none is
// exported.
#ifndef HC_AMD_INTERNAL_H
#define HC_AMD_INTERNAL_H

#include "hc_amd_runtime.h"

#define HCAMD_HIDDEN __attribute__((visibility("hidden")))

extern "C" {
// runtime.cpp: the HIP device index a queue runs on (-1 for a null queue), and
// the queue's error callback with a printf-style message.
HCAMD_HIDDEN int hcamdInternalQueueDeviceIndex(OlQueue q) noexcept;
HCAMD_HIDDEN void hcamdInternalReport(OlQueue q, const char *fmt, ...) noexcept
    __attribute__((format(printf, 2, 3)));
// runtime.cpp: whether the column-reduction kernels of the queue's device were
// resolved when the device was created (a launch then loads nothing).
HCAMD_HIDDEN int hcamdInternalColsKernelsReady(OlQueue q) noexcept;

// scratch.hip: looks up the address of the library's static device scratch
// array on `device`, which must be current; 0 on success, else the HIP error
// name in `err`.  Called once per device by olCreateDevice.
HCAMD_HIDDEN int hcamdInternalScratchSetup(int device, char *err, size_t errLen) noexcept;
}

#endif
