/*
 * Copies between caller-owned (pageable) host memory and device memory.
 *
 * The reference registers the caller's memory with the driver and lets the
 * device read it in place (gpu_memory_cuda.cpp:811-820, with a staged copy as
 * the fallback). Registration of existing memory is not available on the
 * target machines, and a plain hipMemcpy from pageable memory is staged by the
 * runtime on one thread (measured 30 GB/s up, 18 GB/s down, against 57 GB/s
 * for pinned memory in either direction). These routines do the staging
 * themselves: a ring of pinned chunks, filled or drained by a few host threads
 * while the DMA engine moves the neighbouring chunk.
 *
 * Both calls are ordered on `stream` like an asynchronous copy:
 *  - upload returns once the host source has been read completely (the caller
 *    may overwrite it); the last chunks may still be in flight on `stream`;
 *  - download returns once the host destination is complete.
 * The ring is shared: calls must not overlap (the callers hold the runtime's
 * device mutex).
 */
#pragma once
#include <hip/hip_runtime.h>
#include <cstddef>

int eshkol_hip_upload(void* dev, const void* host, size_t bytes, hipStream_t stream);
int eshkol_hip_download(void* host, const void* dev, size_t bytes, hipStream_t stream);

/* Frees the pinned ring and its events (the worker threads stay parked). */
void eshkol_hip_copy_release(void);
