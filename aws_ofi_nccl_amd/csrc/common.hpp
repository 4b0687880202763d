/*
 * Shared host-side helpers of libofi_amd_hotpath.so: HIP error -> errno
 * translation (the convention of include/nccl_ofi_rocm.h in the reference),
 * device presence check, and the pinned-host word kernels use to report a
 * precondition violation they detected on the device.
 */
#ifndef OFI_AMD_COMMON_HPP_
#define OFI_AMD_COMMON_HPP_

#include <cerrno>
#include <cstdint>
#include <cstdio>

#include <hip/hip_runtime.h>

namespace ofi_amd {

inline int errno_of(hipError_t e)
{
	switch (e) {
	case hipSuccess: return 0;
	case hipErrorNoDevice:
	case hipErrorInvalidDevice:
	case hipErrorInsufficientDriver: return -ENODEV;
	case hipErrorOutOfMemory: return -ENOMEM;
	case hipErrorInvalidValue:
	case hipErrorInvalidDevicePointer: return -EINVAL;
	case hipErrorNotSupported: return -ENOTSUP;
	default: return -EIO;
	}
}

/* A failed call is reported through the return value only: the runtime's per-thread
 * "last error" is cleared so that it does not surface in an unrelated later call of the
 * application (hipGetLastError / hipPeekAtLastError users). */
#define OFI_AMD_HIP_TRY(expr)                                                           \
	do {                                                                            \
		hipError_t e_ = (expr);                                                 \
		if (e_ != hipSuccess) {                                                 \
			(void)hipGetLastError();                                        \
			return ::ofi_amd::errno_of(e_);                                 \
		}                                                                       \
	} while (0)

/* 0 when at least one GPU is usable, else -ENODEV.  Never falls back. */
int require_device();

/* Device-visible error word (pinned host memory): kernels OR a bit into it when
 * they skip work because a documented precondition does not hold. */
uint32_t *async_error_word();
/* The same word if ofi_amd_gpu_init() or an earlier call has already allocated it, else
 * NULL: for entry points that must not allocate. */
uint32_t *async_error_word_if_ready();

/* Looks up, for every GPU, the device address of the striping scratch that
 * ofi_amd_sched_batch_noalloc uses.  Called by ofi_amd_gpu_init(). */
int sched_noalloc_setup();

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

enum : uint32_t {
	ASYNC_ERR_BOUNCE_RANGE = 1u << 0, /* destination range outside arena or misaligned */
	ASYNC_ERR_GIN_TIMEOUT = 1u << 1,  /* producer gave up on a full ring */
	ASYNC_ERR_SCHED_STATE = 1u << 2,  /* scheduler state unusable (rails, stripe size) */
	ASYNC_ERR_COPY_LENGTH = 1u << 3,  /* a copy-table entry longer than the stated maximum */
};

/* The device side of a flush read for the first 64 lanes of a workgroup: one lane per 8-byte
 * word, 8 words per rail slot.  The flag (word 0 of a slot) is what the host polls, so it goes
 * last, behind a system-scope release fence. */
__device__ __forceinline__ void flush_post_lanes(const uint64_t *__restrict__ flush_buf, uint64_t *__restrict__ slots,
						 uint32_t num_rails, uint32_t lane)
{
	const uint32_t rail = lane >> 3, word = lane & 7u;
	if (rail >= num_rails) {
		return;
	}
	const uint64_t v = __hip_atomic_load(&flush_buf[word], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM);
	if (word != 0) {
		__hip_atomic_store(&slots[rail * 8u + word], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
	}
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
	if (word == 0) {
		__hip_atomic_store(&slots[rail * 8u], v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
	}
}

} // namespace ofi_amd

#endif
