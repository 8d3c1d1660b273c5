/*
 * nvshmem.h - OpenSHMEM-standard part of the NVSHMEM data-movement API, MI355X logical-PE build.
 * Host C ABI for every compiler; device API (inline, gfx950) when compiled by hipcc.
 * Stands where the reference's src/include/nvshmem.h:15-29 stands.
 */
#ifndef NVSHMEM_H
#define NVSHMEM_H

#include "nvshmem_amd/nvshmem_constants.h"
#include "nvshmem_amd/nvshmem_types.h"
#include "nvshmem_amd/nvshmem_host_api.h"

#if defined(__HIPCC__)
#include "nvshmem_amd/device/nvshmem_device_api.h"
#endif

#endif
