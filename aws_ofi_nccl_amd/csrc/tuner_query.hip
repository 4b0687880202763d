/*
 * Point queries of the tuner: a list of independent questions (region decision, model
 * decision, chunk size) answered by one launch, one thread per question.  The tuner
 * plugin's per-collective entry points are served from here through a cache
 * (tuner_plugin.cpp); irregular batch callers can use it directly.
 */
#include <cstring>
#include <mutex>

#include "common.hpp"
#include "tuner_device.hpp"

using namespace ofi_amd_tuner;

namespace {

/* device form of one question: the public fields plus log2 coordinates from host libm */
struct dev_query_t {
	ofi_amd_tuner_query_t q;
	double log2_bytes;
	double log2_ranks;
	double log2_nodes;
};

__global__ __launch_bounds__(64) void tuner_query_kernel(region_tables_t t,
							 const dev_query_t *__restrict__ queries, uint32_t n,
							 ofi_amd_tuner_answer_t *__restrict__ answers)
{
	const uint32_t i = blockIdx.x * 64u + threadIdx.x;
	if (i >= n) {
		return;
	}
	const dev_query_t d = queries[i];
	const ofi_amd_tuner_query_t &q = d.q;
	int algo = -1, proto = -1, nch = -1;
	uint64_t chunk = 0;
	switch (q.kind) {
	case 0:
		region_choose(t, q.platform, q.coll, q.nbytes, q.num_ranks, q.num_nodes,
			      pt_t{ d.log2_bytes, d.log2_ranks }, q.allowed_mask, algo, proto, nch);
		break;
	case 1:
		model_choose(q.platform, q.coll, q.nbytes, q.num_ranks, q.num_nodes, d.log2_nodes,
			     q.pipe_ops, q.num_channels, q.net_comp_overhead, q.allowed_mask, algo, proto);
		break;
	case 2:
		chunk = region_chunk_size(q.platform, q.coll, q.nbytes, q.algo, q.proto, q.num_ranks,
					  q.num_nodes);
		break;
	default:
		break;
	}
	ofi_amd_tuner_answer_t a;
	a.algo = (int8_t)algo;
	a.proto = (int8_t)proto;
	a.nchannels = (int16_t)nch;
	a.pad = 0;
	a.chunk_size = chunk;
	answers[i] = a;
}

/* Pinned staging for questions and answers plus a private stream, grown on demand. */
struct staging_t {
	std::mutex lock;
	dev_query_t *q = nullptr;           /* pinned host, device-visible */
	ofi_amd_tuner_answer_t *a = nullptr; /* pinned host, device-visible */
	uint32_t cap = 0;
	hipStream_t stream = nullptr;
};
/* one per GPU: a stream and pinned staging belong to the device that was current when they
 * were made, and a process may drive several */
constexpr int kMaxDevices = 64;
staging_t g_stages[kMaxDevices];

staging_t *stage_of_current_device()
{
	int dev = -1;
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
		(void)hipGetLastError();
		return nullptr;
	}
	return &g_stages[dev];
}

} // namespace

/* stream and staging for `want` questions; the caller holds g_stage.lock */
static int ensure_staging(staging_t &g_stage, uint32_t want)
{
	if (!g_stage.stream) {
		OFI_AMD_HIP_TRY(hipStreamCreateWithFlags(&g_stage.stream, hipStreamNonBlocking));
	}
	if (want > g_stage.cap) {
		want = want < 256 ? 256 : want;
		void *q = nullptr, *a = nullptr;
		OFI_AMD_HIP_TRY(hipHostMalloc(&q, sizeof(dev_query_t) * want, hipHostMallocMapped));
		if (hipHostMalloc(&a, sizeof(ofi_amd_tuner_answer_t) * want, hipHostMallocMapped) != hipSuccess) {
			(void)hipGetLastError();
			(void)hipHostFree(q);
			return -ENOMEM;
		}
		if (g_stage.q) (void)hipHostFree(g_stage.q);
		if (g_stage.a) (void)hipHostFree(g_stage.a);
		g_stage.q = static_cast<dev_query_t *>(q);
		g_stage.a = static_cast<ofi_amd_tuner_answer_t *>(a);
		g_stage.cap = want;
	}
	return 0;
}

using namespace ofi_amd;

extern "C" int ofi_amd_tuner_query_prepare(uint32_t capacity)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	region_tables_t tables;
	rc = device_region_tables(&tables);
	if (rc != 0) {
		return rc;
	}
	staging_t *stage = stage_of_current_device();
	if (!stage) {
		return -ENODEV;
	}
	std::lock_guard<std::mutex> g(stage->lock);
	return ensure_staging(*stage, capacity);
}

extern "C" int ofi_amd_tuner_query(const ofi_amd_tuner_query_t *queries, uint32_t n,
				   ofi_amd_tuner_answer_t *answers)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (n == 0) {
		return 0;
	}
	if (!queries || !answers) {
		return -EINVAL;
	}
	for (uint32_t i = 0; i < n; i++) {
		const ofi_amd_tuner_query_t &q = queries[i];
		if (q.platform < 0 || q.platform >= kNumPlatforms || q.kind < 0 || q.kind > 2 ||
		    q.num_nodes == 0 || q.num_ranks == 0 || q.coll < 0) {
			return -EINVAL;
		}
		if (q.kind == 2 && (q.algo < 0 || q.algo >= NUM_ALGOS || q.proto < 0 || q.proto >= NUM_PROTOS)) {
			return -EINVAL;
		}
	}
	region_tables_t tables;
	rc = device_region_tables(&tables);
	if (rc != 0) {
		return rc;
	}

	staging_t *stage = stage_of_current_device();
	if (!stage) {
		return -ENODEV;
	}
	staging_t &g_stage = *stage;
	std::lock_guard<std::mutex> g(g_stage.lock);
	rc = ensure_staging(g_stage, n);
	if (rc != 0) {
		return rc;
	}
	for (uint32_t i = 0; i < n; i++) {
		dev_query_t &d = g_stage.q[i];
		d.q = queries[i];
		d.log2_bytes = log2_coord((double)queries[i].nbytes);
		d.log2_ranks = log2_coord((double)queries[i].num_ranks);
		d.log2_nodes = std::log2((double)queries[i].num_nodes);
	}
	void *dq = nullptr, *da = nullptr;
	OFI_AMD_HIP_TRY(hipHostGetDevicePointer(&dq, g_stage.q, 0));
	OFI_AMD_HIP_TRY(hipHostGetDevicePointer(&da, g_stage.a, 0));
	hipLaunchKernelGGL(tuner_query_kernel, dim3((n + 63) / 64), dim3(64), 0, g_stage.stream, tables,
			   static_cast<const dev_query_t *>(dq), n, static_cast<ofi_amd_tuner_answer_t *>(da));
	OFI_AMD_HIP_TRY(hipGetLastError());
	OFI_AMD_HIP_TRY(hipStreamSynchronize(g_stage.stream));
	std::memcpy(answers, g_stage.a, sizeof(ofi_amd_tuner_answer_t) * n);
	return 0;
}
