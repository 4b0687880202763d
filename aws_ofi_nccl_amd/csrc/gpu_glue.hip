/*
 * GPU runtime glue behind the C ABI: the MI355X replacement for
 * src/nccl_ofi_rocm.cpp of the reference (which stubs flush and device lookup)
 * plus the calls that only the reference's CUDA build has and that GIN needs
 * (include/nccl_ofi_cuda.h:34-139).  Negative errno on failure.
 */
#include <atomic>
#include <cstring>
#include <mutex>

#include <unistd.h>

#include "common.hpp"
#include "ofi_amd_hotpath.h"

namespace ofi_amd {

int require_device()
{
	static std::once_flag once;
	static int status = -ENODEV;
	std::call_once(once, [] {
		int count = 0;
		hipError_t e = hipGetDeviceCount(&count);
		status = (e == hipSuccess && count > 0) ? 0 : -ENODEV;
	});
	return status;
}

namespace {
std::atomic<uint32_t *> g_async_error_word{nullptr};
}

uint32_t *async_error_word()
{
	static std::once_flag once;
	std::call_once(once, [] {
		void *p = nullptr;
		if (hipHostMalloc(&p, 64, hipHostMallocMapped) == hipSuccess) {
			std::memset(p, 0, 64);
			g_async_error_word.store(static_cast<uint32_t *>(p), std::memory_order_release);
		}
	});
	return g_async_error_word.load(std::memory_order_acquire);
}

uint32_t *async_error_word_if_ready()
{
	return g_async_error_word.load(std::memory_order_acquire);
}

} // namespace ofi_amd

using namespace ofi_amd;

extern "C" {

int ofi_amd_gpu_init(void)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	int driver = -1, runtime = -1;
	OFI_AMD_HIP_TRY(hipDriverGetVersion(&driver));
	OFI_AMD_HIP_TRY(hipRuntimeGetVersion(&runtime));
	if (!async_error_word()) {
		return -ENOMEM;
	}
	return sched_noalloc_setup();
}

int ofi_amd_async_error_fetch(uint32_t *bits)
{
	uint32_t *w = async_error_word();
	if (!w || !bits) {
		return -EINVAL;
	}
	*bits = __atomic_exchange_n(w, 0u, __ATOMIC_ACQ_REL);
	return 0;
}

int ofi_amd_gpu_get_device_for_addr(void *data, int *dev_id)
{
	if (!dev_id) {
		return -EINVAL;
	}
	*dev_id = -1;
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	hipPointerAttribute_t attr;
	if (hipPointerGetAttributes(&attr, data) != hipSuccess) {
		(void)hipGetLastError();
		return -ENOTSUP;
	}
	if (attr.type != hipMemoryTypeDevice && attr.type != hipMemoryTypeManaged) {
		return -ENOTSUP;
	}
	*dev_id = attr.device;
	return 0;
}

int ofi_amd_gpu_flush_gpudirect_rdma_writes(void)
{
	return -EPERM;
}

int ofi_amd_gpu_mem_alloc(void **ptr, size_t size)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	OFI_AMD_HIP_TRY(hipMalloc(ptr, size));
	return 0;
}

int ofi_amd_gpu_mem_free(void *ptr)
{
	OFI_AMD_HIP_TRY(hipFree(ptr));
	return 0;
}

int ofi_amd_gpu_mem_copy_host_to_device(void *dst, const void *src, size_t size)
{
	OFI_AMD_HIP_TRY(hipMemcpy(dst, src, size, hipMemcpyHostToDevice));
	return 0;
}

int ofi_amd_gpu_mem_copy_device_to_host(void *dst, const void *src, size_t size)
{
	OFI_AMD_HIP_TRY(hipMemcpy(dst, src, size, hipMemcpyDeviceToHost));
	return 0;
}

int ofi_amd_gpu_stream_synchronize(void *stream)
{
	OFI_AMD_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
	return 0;
}

int ofi_amd_gpu_get_dma_buf_fd(void *aligned_ptr, size_t aligned_size, int *fd, size_t *offset)
{
	if (!fd || !offset) {
		return -EINVAL;
	}
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	OFI_AMD_HIP_TRY(hipMemGetHandleForAddressRange(fd, (hipDeviceptr_t)aligned_ptr, aligned_size,
						       hipMemRangeHandleTypeDmaBufFd, 0));
	*offset = 0;
	return 0;
}

int ofi_amd_gpu_have_dma_buf_attr(void)
{
	if (require_device() != 0) {
		return 0;
	}
	int dev = 0, supported = 0;
	if (hipGetDevice(&dev) != hipSuccess) {
		return 0;
	}
	/* Probe rather than query: export a dma-buf for a small allocation. */
	static std::once_flag once;
	static int cached = 0;
	std::call_once(once, [&] {
		void *p = nullptr;
		if (hipMalloc(&p, 1 << 16) != hipSuccess) {
			return;
		}
		int fd = -1;
		if (hipMemGetHandleForAddressRange(&fd, (hipDeviceptr_t)p, 1 << 16,
						   hipMemRangeHandleTypeDmaBufFd, 0) == hipSuccess &&
		    fd >= 0) {
			cached = 1;
			close(fd);
		} else {
			(void)hipGetLastError();
		}
		(void)hipFree(p);
	});
	supported = cached;
	return supported;
}

int ofi_amd_gpu_have_gdr_support_attr(void)
{
	return 0; /* src/nccl_ofi_rocm.cpp:78-81 */
}

int ofi_amd_gpu_set_current_device(int dev_id)
{
	OFI_AMD_HIP_TRY(hipSetDevice(dev_id));
	return 0;
}

int ofi_amd_gpu_get_current_device(int *dev_id)
{
	if (!dev_id) {
		return -EINVAL;
	}
	OFI_AMD_HIP_TRY(hipGetDevice(dev_id));
	return 0;
}

int ofi_amd_gpu_get_address_range(void *ptr, void **base_out, size_t *size_out)
{
	if (!base_out || !size_out) {
		return -EINVAL;
	}
	hipDeviceptr_t base = nullptr;
	size_t size = 0;
	OFI_AMD_HIP_TRY(hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)ptr));
	*base_out = (void *)base;
	*size_out = size;
	return 0;
}

int ofi_amd_gpu_seg_is_host(void *seg_base, int *is_host_out)
{
	if (!is_host_out) {
		return -EINVAL;
	}
	hipPointerAttribute_t attr;
	if (hipPointerGetAttributes(&attr, seg_base) != hipSuccess) {
		(void)hipGetLastError();
		/* unknown to the runtime: ordinary pageable host memory */
		*is_host_out = 1;
		return 0;
	}
	*is_host_out = (attr.type == hipMemoryTypeHost || attr.type == hipMemoryTypeUnregistered) ? 1 : 0;
	return 0;
}

int ofi_amd_gpu_host_alloc(void **ptr, size_t size)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	OFI_AMD_HIP_TRY(hipHostMalloc(ptr, size, hipHostMallocMapped | hipHostMallocCoherent));
	return 0;
}

int ofi_amd_gpu_host_free(void *ptr)
{
	OFI_AMD_HIP_TRY(hipHostFree(ptr));
	return 0;
}

int ofi_amd_gpu_host_get_device_pointer(void **dev_ptr, void *host_ptr)
{
	OFI_AMD_HIP_TRY(hipHostGetDevicePointer(dev_ptr, host_ptr, 0));
	return 0;
}

} /* extern "C" */
