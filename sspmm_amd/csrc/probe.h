// Diagnostic kernels of the library (see probe.hip).
#ifndef SSPMM_AMD_PROBE_H
#define SSPMM_AMD_PROBE_H

#include <hip/hip_runtime.h>

namespace sspmm {

// waves x steps x 8 KiB of 16-byte gathers from a [rows x row_bytes] matrix (row_bytes a multiple of 256);
// sink: at least 16 bytes per wave, never written in practice.
hipError_t launch_probe_gather(const void *matrix, int rows, int row_bytes, int waves, int steps, void *sink,
                               hipStream_t stream);

}  // namespace sspmm
#endif
