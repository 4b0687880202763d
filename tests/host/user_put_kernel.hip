/*
 * What a user of include/ofi_amd_gin_device.h writes: a kernel of their own that initiates
 * puts.  Compiled (not run) by tests/test_abi_host.py to show the header stands on its own.
 */
#include "ofi_amd_gin_device.h"

__global__ void user_put_kernel(ofi_amd_gin_dev_ring_t ring, const uint64_t *dst_offsets, uint32_t n,
				int *status)
{
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	ofi_amd_gin_desc_t d = {};
	d.size = 8;
	d.dst_off = i < n ? dst_offsets[i] : 0;
	d.rank = 1;
	d.dst_mr = 1;
	d.sig_mr = 0xffff;
	d.context = ring.context;
	/* every lane of the wavefront makes the call; only the first n threads put */
	if (ofi_amd_gin_dev_put(ring, &d, i < n, 1u << 20) != 0 && (threadIdx.x & 63u) == 0) {
		*status = -1;
	}
}
