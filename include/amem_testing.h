/*
 * amem_testing.h — measurement and test helpers exported by libamem_nccl.so.1 beside the product
 * surface of amem.h. None of them has a counterpart in the reference and none is needed by a
 * caller of the pause/resume path: they exist so that tests and the benchmark can move bytes,
 * read device state and measure the platform through the same library, without a second one.
 * Plain C like amem.h.
 */
#ifndef AMEM_TESTING_H_
#define AMEM_TESTING_H_

#include "amem.h"

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

/* Measured host-link roofline: best-of-`reps` hipMemcpy of `bytes` between device memory
 * and a pinned host buffer, each direction, in GB/s (1e9 bytes per second). */
int amem_probe_link(uint64_t bytes, int reps, double* d2h_gbps, double* h2d_gbps);

/* What one hipMemUnmap costs on this machine with nothing else running: `count` mappings of `bytes`
 * each are created, mapped and made accessible; the device is idle; each is then unmapped, timed on
 * its own. Writes the median and the mean time of one call in microseconds (either may be NULL), and
 * the mean time of one create + map + set-access triple. Everything is released again. 0, or a HIP error. */
int amem_probe_unmap(int count, uint64_t bytes, double* unmap_us_p50, double* unmap_us_mean, double* map_us_mean);

/* Plain device-to-device copy kernel of `bytes` (multiple of 16), used to calibrate the
 * FETCH_SIZE / WRITE_SIZE hardware counters against a known traffic. */
int amem_calib_copy(uint64_t bytes, int reps, float* kernel_ms);

/* Raw byte access (hipMemcpy wrappers, synchronous). */
int amem_copy_to_device(uint64_t va, const void* host, uint64_t bytes);
int amem_copy_from_device(void* host, uint64_t va, uint64_t bytes);
int amem_device_mem_info(uint64_t* free_bytes, uint64_t* total_bytes);
int amem_device_count(void);
/* PCI address of the current device as "dddd:bb:dd.f" (for looking its NUMA node up in sysfs). */
int amem_device_pci_bus_id(char* out, int len);

#pragma GCC visibility pop
#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* AMEM_TESTING_H_ */
