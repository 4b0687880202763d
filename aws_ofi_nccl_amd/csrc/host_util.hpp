/*
 * Small host-side helpers shared by the in-process fabrics and links: pinned host memory the GPU
 * reads and writes in place, and a fixed-size queue.
 */
#ifndef OFI_AMD_HOST_UTIL_HPP_
#define OFI_AMD_HOST_UTIL_HPP_

#include <cstdint>
#include <cstring>
#include <vector>

#include "ofi_amd_hotpath.h"

namespace ofi_amd {

/* Pinned host memory (zeroed) and the address the GPU reaches it by. */
struct pinned_t {
	void *host = nullptr;
	void *dev = nullptr;
	int alloc(size_t bytes)
	{
		const size_t n = bytes ? bytes : 8;
		int rc = ofi_amd_gpu_host_alloc(&host, n);
		if (rc == 0) {
			std::memset(host, 0, n);
			rc = ofi_amd_gpu_host_get_device_pointer(&dev, host);
		}
		return rc;
	}
	void release()
	{
		if (host) {
			(void)ofi_amd_gpu_host_free(host);
		}
		host = dev = nullptr;
	}
	template <typename T> T *as() { return static_cast<T *>(host); }
	template <typename T> const T *dev_as() const { return static_cast<const T *>(dev); }
};

/* Fixed-size queue over a power-of-two array: positions only grow, the index is the position
 * masked. */
template <typename T>
struct ring_t {
	std::vector<T> slot;
	uint32_t mask = 0, head = 0, tail = 0; /* head: oldest entry, tail: next free position */
	void reset(uint32_t capacity)
	{
		uint32_t n = 1;
		while (n < capacity) {
			n <<= 1;
		}
		slot.assign(n, T());
		mask = n - 1;
		head = tail = 0;
	}
	uint32_t size() const { return tail - head; }
	bool empty() const { return tail == head; }
	T &at(uint32_t k) { return slot[(head + k) & mask]; } /* k-th oldest */
	void push(const T &v) { slot[tail++ & mask] = v; }
	void pop() { head++; }
};

} // namespace ofi_amd

#endif
