#pragma once
// Host-side interface of the device code that is compiled into the library ahead of time
// (src/device_code.hip). Internal: reached through the C ABI of qmlp_hip.h / qmlp_capi.h only.

#include <cstddef>
#include <string>

/** Size of the static device buffer behind qmlp_network_inference_noalloc (per GPU). */
#define QMLP_STATIC_SCRATCH_BYTES (48u << 20)

namespace qmlp { namespace device_code {

/** Fills `bytes` bytes at `ptr` (device memory) with `value` by a kernel on `stream`. Returns 0 or sets `error`. */
int fillAsync(void* ptr, int value, size_t bytes, void* stream, std::string& error);

/**
 * Address of the current device's copy of the static scratch buffer and its size. The first
 * call on a device resolves the address (which loads the library's code object onto that
 * device); later calls only read it. Returns 0 or sets `error`.
 */
int staticScratch(void** ptr, size_t* bytes, std::string& error);

/**
 * Notes that work on `stream` is about to use the static scratch buffer of the current device. All calls on a
 * device share the buffer: a call on another stream than the last one is accepted only if that stream's work has
 * finished (and this stream is not being captured, when other streams may not be asked). Allocates nothing.
 * Returns 0 or sets `error`.
 */
int claimStaticScratch(void* stream, std::string& error);

}} // namespace qmlp::device_code
