/*
 * dflash_profile.h -- measurement hooks of libdflash_hip.so.
 *
 * NOT part of the drop-in surface (include/dflash_hip.h, include/dflash_cache.h): nothing the reference's call
 * sites need is declared here, the module map does not export this header, and a host that only serves requests
 * never includes it.  The benchmark and the profiles use these two entries to time single kernels and to price a
 * launch that does no work.
 */
#ifndef DFLASH_PROFILE_H
#define DFLASH_PROFILE_H

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------
 * Measurement hook (no counterpart in the reference, whose bench times whole
 * calls from the host: Sources/DFlashKernelBench/main.swift:33-57).  Arms the
 * calling thread so that the NEXT launch of the named kernel carries the two
 * events on its own dispatch (hipExtLaunchKernelGGL): their elapsed time is the
 * kernel's begin-to-end duration on the launch stream, as a profiler's kernel
 * trace reports it.  The arming is consumed by that launch.  Events are
 * hipEvent_t passed as void*, created and read by the caller.
 * ---------------------------------------------------------------------- */
#define DFLASH_KERNEL_SDPA_PARTIAL 0
#define DFLASH_KERNEL_SDPA_COMBINE 1
#define DFLASH_KERNEL_GDN_FORWARD 2
#define DFLASH_KERNEL_TAPE_REPLAY 3
#define DFLASH_KERNEL_GREEDY_PARTIAL 4
#define DFLASH_KERNEL_GDN_PREPARE 5
#define DFLASH_KERNEL_EMPTY 6
#define DFLASH_KERNEL_GDN_LAYER 7
#define DFLASH_KERNEL_GDN_FINISH 8
#define DFLASH_KERNEL_COUNT 9
int dflash_profile_next_launch(int kernel_id, void* start_event, void* stop_event);

/* Launches a kernel that does nothing, with the given grid, block size (a multiple of 64, at most
 * 1024) and dynamic LDS size (at most 160 KB): the cost of a launch of that shape before any work,
 * i.e. the floor under each kernel of a verify step.  No counterpart in the reference.  Kernel id
 * DFLASH_KERNEL_EMPTY for dflash_profile_next_launch. */
int dflash_profile_empty_launch(void* stream, int grid_x, int grid_y, int grid_z, int threads, int lds_bytes);

#ifdef __cplusplus
}
#endif
#endif /* DFLASH_PROFILE_H */
