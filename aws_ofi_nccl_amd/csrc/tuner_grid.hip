/*
 * Batched tuner evaluation for gfx950: the cost model and the region lookup
 * over a whole grid of (collective, size, nodes, ranks/node) points in one call.
 *
 * Model: nccl_ofi_tuner_compute_cost and model_get_coll_info_internal_v3,
 * src/tuner/nccl_ofi_model.cpp:13-234.  The reference computes in fp32 with two
 * double sub-expressions (log2 of the node count) and never fuses a multiply
 * with an add; the kernels keep every rounding step (this file is built with
 * contraction off, divisions are the correctly rounded ones) and take
 * log2(nodes) precomputed by the host's libm, so costs match bit for bit.
 *
 * Regions: region_get_coll_info_internal_v3, src/tuner/nccl_ofi_regions.cpp:
 * 2070-2157, with is_inside_region (:159-221).  Polygons are built and
 * log2-transformed on the host when the plan is created (:224-289), as are the
 * query coordinates, so the device does no transcendental math.  The one
 * difference from the reference's arithmetic: its `long double` intermediates
 * (:91, :50-56) are 80-bit on x86-64 and plain double here; that can only move a
 * point that lies within ~1e-16 of the 1e-10 on-edge threshold.
 *
 * Nothing here is matrix-shaped: one thread per cost cell (8-byte coalesced
 * stores) and one thread per decision point.
 */
#include <cmath>
#include <cstring>
#include <new>
#include <vector>

#include "common.hpp"
#include "ofi_amd_hotpath.h"
#include "region_tables.inc"

namespace {

/* nccl/tuner.h:14-41 */
enum { FUNC_ALLGATHER = 2, FUNC_REDUCESCATTER = 3, FUNC_ALLREDUCE = 4, NUM_FUNCS = 5 };
enum { ALGO_TREE = 0, ALGO_RING = 1, ALGO_COLLNET_DIRECT = 2, ALGO_COLLNET_CHAIN = 3,
       ALGO_NVLS = 4, ALGO_NVLS_TREE = 5, ALGO_PAT = 6, NUM_ALGOS = 7 };
enum { PROTO_LL = 0, PROTO_LL128 = 1, PROTO_SIMPLE = 2, NUM_PROTOS = 3 };

constexpr int kNumPlatforms = 4;
constexpr int kNumShapes = 3; /* ranks == 8*nodes, 2*nodes, nodes */
constexpr int kMaxVertices = 20;

struct model_params_t {
	float net_lat;
	float internode_bw;
	float intranode_bw;
	int num_rails;
	float nvlink_lat[NUM_ALGOS][NUM_PROTOS];
};

/* src/tuner/nccl_ofi_model.cpp:13-44; the bandwidths are double constant
 * expressions narrowed to float once, as there. */
__constant__ model_params_t c_model_params[2] = {
	{ 20.0f, (float)(12.5 * 1024 * 1024 * 1024 * 1e-6), (float)(20.0 * 1024 * 1024 * 1024 * 1e-6), 4,
	  { { .6f, 1.25f, 28.f }, { .6f, 1.9f, 3.4f }, { 0, 0, 3.7f }, { 0, 0, 2.8f },
	    { 0, 0, 23.f }, { 0, 0, 23.f }, { 0, 0, 0 } } },
	{ 18.0f, (float)(25.0 * 1024 * 1024 * 1024 * 1e-6), (float)(20.0 * 1024 * 1024 * 1024 * 1e-6), 2,
	  { { .6f, 1.25f, 28.f }, { .6f, 1.9f, 3.4f }, { 0, 0, 3.7f }, { 0, 0, 2.8f },
	    { 0, 0, 23.f }, { 0, 0, 23.f }, { 0, 0, 0 } } },
};

struct grid_dims_t {
	uint32_t n_colls, n_sizes, n_nodes, n_ppn, n_algos;
	const int32_t *colls;
	const uint64_t *sizes;
	const uint64_t *nodes;
	const uint32_t *ppn;
	const int32_t *algos;
	const double *log2_nodes; /* log2((double)nodes[i]) from the host's libm */
};

/* nccl_ofi_tuner_compute_cost, src/tuner/nccl_ofi_model.cpp:46-122 */
__device__ float model_cost(const model_params_t &params, int coll, int algo, int proto,
			    int pipe_ops, uint64_t size, uint64_t num_ranks, uint64_t num_nodes,
			    double log2_nodes, int num_channels, int net_comp_overhead)
{
	if (coll != FUNC_ALLREDUCE) {
		return -1.0f;
	}
	const float net_lat = (proto == PROTO_SIMPLE)
				      ? __fadd_rn(params.net_lat, (float)net_comp_overhead)
				      : params.net_lat;
	const float p2p_lat = params.nvlink_lat[algo][proto];
	float latency, bw;

	switch (algo) {
	case ALGO_RING: {
		int num_steps = (int)(2 * (num_ranks - 1));
		int num_internode_steps = (int)(2 * num_nodes);
		latency = __fadd_rn(__fmul_rn((float)num_internode_steps, net_lat),
				    __fmul_rn((float)(num_steps - num_internode_steps), p2p_lat));
		bw = __fmul_rn(__fmul_rn(params.internode_bw, (float)params.num_rails),
			       (float)num_channels);
		break;
	}
	case ALGO_NVLS_TREE: {
		double t = __dadd_rn((double)p2p_lat, __dmul_rn(log2_nodes, (double)net_lat));
		latency = (float)__dmul_rn(2.0, t);
		float half = __fdiv_rn(__fmul_rn(params.internode_bw, (float)params.num_rails), 2.0f);
		bw = __fmul_rn(half < params.intranode_bw ? half : params.intranode_bw,
			       (float)num_channels);
		break;
	}
	case ALGO_TREE: {
		float a = __fmul_rn((float)(2 * ((num_ranks / num_nodes) - 1)), p2p_lat);
		double b = __dmul_rn(__dmul_rn(2.0, log2_nodes), (double)net_lat);
		latency = (float)__dadd_rn((double)a, b);
		bw = __fdiv_rn(__fmul_rn(__fmul_rn(params.internode_bw, (float)params.num_rails),
					 (float)num_channels),
			       2.0f);
		break;
	}
	default:
		return -1.0f;
	}

	if (proto == PROTO_LL) {
		bw = (float)__dmul_rn((double)bw, 0.5);
	} else if (proto == PROTO_LL128) {
		bw = (float)__dmul_rn((double)bw, 0.9375);
	}
	return __fadd_rn(__fmul_rn(latency, (float)pipe_ops), __fdiv_rn((float)size, bw));
}

/* One thread per cost cell. */
__global__ __launch_bounds__(256) void model_cost_kernel(grid_dims_t g,
							 const ofi_amd_tuner_variant_t *__restrict__ variants,
							 uint32_t n_variants, uint64_t cells_per_variant,
							 double *__restrict__ cost)
{
	const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
	if (idx >= cells_per_variant * n_variants) {
		return;
	}
	uint64_t r = idx;
	const uint32_t proto = (uint32_t)(r % NUM_PROTOS); r /= NUM_PROTOS;
	const uint32_t ai = (uint32_t)(r % g.n_algos); r /= g.n_algos;
	const uint32_t pi = (uint32_t)(r % g.n_ppn); r /= g.n_ppn;
	const uint32_t ni = (uint32_t)(r % g.n_nodes); r /= g.n_nodes;
	const uint32_t si = (uint32_t)(r % g.n_sizes); r /= g.n_sizes;
	const uint32_t ci = (uint32_t)(r % g.n_colls); r /= g.n_colls;
	const ofi_amd_tuner_variant_t v = variants[r];

	const uint64_t nodes = g.nodes[ni];
	const uint64_t ranks = nodes * g.ppn[pi];
	float c = -1.0f;
	if (v.platform == OFI_AMD_PLATFORM_P5_P5E || v.platform == OFI_AMD_PLATFORM_P5EN) {
		c = model_cost(c_model_params[v.platform], g.colls[ci], g.algos[ai], (int)proto,
			       v.pipe_ops, g.sizes[si], ranks, nodes, g.log2_nodes[ni],
			       v.num_channels, v.net_comp_overhead);
	}
	cost[idx] = (double)c;
}

/* One thread per decision point: model_get_coll_info_internal_v3, :154-234. */
__global__ __launch_bounds__(256) void model_choice_kernel(grid_dims_t g,
							   const ofi_amd_tuner_variant_t *__restrict__ variants,
							   uint32_t n_variants, uint64_t points_per_variant,
							   int8_t *__restrict__ choice)
{
	const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
	if (idx >= points_per_variant * n_variants) {
		return;
	}
	uint64_t r = idx;
	const uint32_t pi = (uint32_t)(r % g.n_ppn); r /= g.n_ppn;
	const uint32_t ni = (uint32_t)(r % g.n_nodes); r /= g.n_nodes;
	const uint32_t si = (uint32_t)(r % g.n_sizes); r /= g.n_sizes;
	const uint32_t ci = (uint32_t)(r % g.n_colls); r /= g.n_colls;
	const ofi_amd_tuner_variant_t v = variants[r];

	const uint64_t nodes = g.nodes[ni];
	const uint64_t ranks = nodes * g.ppn[pi];
	const uint64_t size = g.sizes[si];
	const int coll = g.colls[ci];
	int chosen_algo = -1, chosen_proto = -1;

	const bool modelled = v.platform == OFI_AMD_PLATFORM_P5_P5E || v.platform == OFI_AMD_PLATFORM_P5EN;
	if (modelled && nodes > 2) { /* :178 */
		if (v.platform == OFI_AMD_PLATFORM_P5_P5E && coll == FUNC_ALLREDUCE && nodes == 16 &&
		    ranks == 128 && size > 3ULL * 1024 * 1024 * 1024 && size <= 5ULL * 1024 * 1024 * 1024) {
			chosen_algo = ALGO_NVLS_TREE; /* :183-192 */
			chosen_proto = PROTO_SIMPLE;
		} else {
			float lowest = 3.402823466e+38f; /* FLT_MAX */
			for (int algo = 0; algo < NUM_ALGOS; algo++) {
				if (algo == ALGO_COLLNET_DIRECT || algo == ALGO_COLLNET_CHAIN || algo == ALGO_NVLS) {
					continue;
				}
				for (int proto = 0; proto < NUM_PROTOS; proto++) {
					if (algo == ALGO_NVLS_TREE && proto != PROTO_SIMPLE) {
						continue;
					}
					float c = model_cost(c_model_params[v.platform], coll, algo, proto,
							     v.pipe_ops, size, ranks, nodes, g.log2_nodes[ni],
							     v.num_channels, v.net_comp_overhead);
					if (c < 0) {
						continue;
					}
					if (c < lowest) {
						chosen_algo = algo;
						chosen_proto = proto;
						lowest = c;
					}
				}
			}
		}
	}
	choice[idx * 2 + 0] = (int8_t)chosen_algo;
	choice[idx * 2 + 1] = (int8_t)chosen_proto;
}

/* ------------------------------------------------------------------ regions */

struct pt_t {
	double x, y;
};

struct region_tables_t {
	/* [platform][shape][coll] -> first polygon / count, -1 when no regions */
	int32_t set_first[kNumPlatforms][kNumShapes][NUM_FUNCS];
	int32_t set_count[kNumPlatforms][kNumShapes][NUM_FUNCS];
	const int32_t *poly; /* per polygon {algo, proto, first_vertex, num_vertices} */
	const pt_t *verts;   /* log2 space */
	const double *log2_sizes; /* per size index: transform_log2 of the byte count */
	const double *log2_ranks; /* per (node, ppn): transform_log2 of the rank count */
	pt_t far_point;      /* log2 of (2*max size, 2*max ranks) */
};

__device__ __forceinline__ pt_t vsub(pt_t a, pt_t b) { return pt_t{ a.x - b.x, a.y - b.y }; }
__device__ __forceinline__ double vdot(pt_t a, pt_t b) { return a.x * b.x + a.y * b.y; }
__device__ __forceinline__ double vcross(pt_t a, pt_t b) { return a.x * b.y - a.y * b.x; }

/* intersect, src/tuner/nccl_ofi_regions.cpp:77-109 */
__device__ int intersect(pt_t x0, pt_t x1, pt_t y0, pt_t y1, double eps, pt_t *sect)
{
	pt_t dx = vsub(x1, x0);
	pt_t dy = vsub(y1, y0);
	double d = vcross(dy, dx);
	if (fabs(d) < eps) {
		return 0;
	}
	double a = (vcross(x0, dx) - vcross(y0, dx)) / d;
	if (sect) {
		sect->x = y0.x + a * dy.x;
		sect->y = y0.y + a * dy.y;
	}
	if (a < -eps || a > 1 + eps) {
		return -1;
	}
	if (a < eps || a > 1 - eps) {
		return 0;
	}
	a = (vcross(x0, dy) - vcross(y0, dy)) / d;
	if (a < 0 || a > 1) {
		return -1;
	}
	return 1;
}

/* distance, :125-142 */
__device__ double seg_distance(pt_t x, pt_t y0, pt_t y1, double eps)
{
	pt_t dy = vsub(y1, y0);
	pt_t x1, s = { 0, 0 };
	x1.x = x.x + dy.y;
	x1.y = x.y - dy.x;
	int r = intersect(x, x1, y0, y1, eps, &s);
	if (r == -1) {
		return HUGE_VAL;
	}
	s = vsub(s, x);
	return sqrt(vdot(s, s));
}

/* is_inside_region, :159-221 */
__device__ int inside_region(pt_t point, const pt_t *v, int n, pt_t far_point)
{
	const double eps = 1e-10;
	for (int i = 0; i < n; i++) {
		int k = (i + 1) % n;
		if (seg_distance(point, v[i], v[k], eps) < eps) {
			return 0;
		}
	}
	/* y bounds start from vertex 1 as in the reference (:177-178) */
	double min_x = v[0].x, max_x = v[0].x, min_y = v[1].y, max_y = v[1].y;
	for (int i = 0; i < n; i++) {
		if (v[i].x > max_x) max_x = v[i].x;
		if (v[i].x < min_x) min_x = v[i].x;
		if (v[i].y > max_y) max_y = v[i].y;
		if (v[i].y < min_y) min_y = v[i].y;
	}
	if (point.x < min_x || point.x > max_x || point.y < min_y || point.y > max_y) {
		return -1;
	}
	int crosses = 0;
	for (int i = 0; i < n; i++) {
		int k = (i + 1) % n;
		if (intersect(point, far_point, v[i], v[k], eps, nullptr) == 1) {
			crosses++;
		}
	}
	return (crosses & 1) ? 1 : -1;
}

/* calculateChunkSizeTreeLL128, :1883-1938 (constants: include/internal/tuner/nccl_defaults.h) */
__device__ uint64_t chunk_tree_ll128(uint64_t message_size, int nChannels, int log2_nnodes)
{
	const int ppn = 8;
	const uint64_t STEPS = 8, ELEMS_PER_THREAD = 120, MAX_NTHREADS = 640;
	const uint64_t LINEELEMS = 16, DATAELEMS = 15, WARP = 32, SHMEM_ELEMS = 8;

	uint64_t buffSize = ELEMS_PER_THREAD * MAX_NTHREADS * STEPS * 8;
	uint64_t chunkSize = buffSize / STEPS;
	chunkSize = (chunkSize / LINEELEMS) * DATAELEMS;
	double nSteps = 1 + log2_nnodes + 0.1 * ppn;

	while ((double)(message_size / ((uint64_t)nChannels * chunkSize)) < nSteps * 64 / ppn &&
	       chunkSize > 131072) {
		chunkSize /= 2;
	}
	while ((double)(message_size / ((uint64_t)nChannels * chunkSize)) < nSteps * 16 / ppn &&
	       chunkSize > 32768) {
		chunkSize /= 2;
	}
	uint64_t grainSize = WARP * SHMEM_ELEMS / LINEELEMS * DATAELEMS * 8;
	chunkSize = (chunkSize / grainSize) * grainSize;
	uint64_t elementsPerGrain = grainSize / 4;
	uint64_t nelem = (chunkSize / grainSize) * elementsPerGrain;
	uint64_t WireWordPerSlice = WARP * SHMEM_ELEMS;
	uint64_t DataEltPerSlice = (WireWordPerSlice - WireWordPerSlice / LINEELEMS) * 2;
	return (uint64_t)(ceil((double)nelem / (double)DataEltPerSlice) * (double)WireWordPerSlice * 8.0);
}

/* One thread per (platform, point): region_get_coll_info_internal_v3, :2070-2157 */
__global__ __launch_bounds__(256) void region_choice_kernel(grid_dims_t g, region_tables_t t,
							    const int32_t *__restrict__ platforms,
							    uint32_t n_platforms,
							    uint64_t points_per_platform,
							    int8_t *__restrict__ choice)
{
	const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
	if (idx >= points_per_platform * n_platforms) {
		return;
	}
	uint64_t r = idx;
	const uint32_t pi = (uint32_t)(r % g.n_ppn); r /= g.n_ppn;
	const uint32_t ni = (uint32_t)(r % g.n_nodes); r /= g.n_nodes;
	const uint32_t si = (uint32_t)(r % g.n_sizes); r /= g.n_sizes;
	const uint32_t ci = (uint32_t)(r % g.n_colls); r /= g.n_colls;
	const int platform = platforms[r];

	const uint64_t nodes = g.nodes[ni];
	const uint32_t ppn = g.ppn[pi];
	const uint64_t ranks = nodes * ppn;
	const uint64_t size = g.sizes[si];
	const int coll = g.colls[ci];

	int algorithm = -1, protocol = -1, nchannels = -1;
	/* shape selection as in the per-platform init functions (:302,:485,:675,:768,:878,...) */
	int shape = -1;
	if (ppn == 8) shape = 0;
	else if (ppn == 2 && platform == OFI_AMD_PLATFORM_P5_P5E) shape = 1;
	else if (ppn == 1) shape = 2;

	if (platform >= 0 && platform < kNumPlatforms && shape >= 0 && coll >= 0 && coll < NUM_FUNCS &&
	    t.set_count[platform][shape][coll] > 0 && nodes > 2) {
		pt_t p = { t.log2_sizes[si], t.log2_ranks[ni * g.n_ppn + pi] };
		const int first = t.set_first[platform][shape][coll];
		const int count = t.set_count[platform][shape][coll];
		int in_out = -1;
		for (int i = 0; i < count && in_out < 0; i++) {
			const int32_t *poly = &t.poly[(first + i) * 4];
			in_out = inside_region(p, &t.verts[poly[2]], poly[3], t.far_point);
			if (in_out >= 0) {
				algorithm = poly[0];
				protocol = poly[1];
			}
		}
		if (in_out >= 0) {
			const int log2_nnodes = 31 - __clz((int)nodes); /* log2i, nccl_defaults.h:92-104 */
			if (platform == OFI_AMD_PLATFORM_P6 && size >= 4 * 1024 * 1024 &&
			    size <= 32 * 1024 * 1024 && algorithm == ALGO_TREE && protocol == PROTO_LL128 &&
			    nodes * 8 == ranks) { /* :2140-2146 */
				const int channels[3] = { 16, 24, 32 };
				int best = 0;
				uint64_t max_chunk = 0;
				for (int c = 0; c < 3; c++) { /* calculateBestNChannelTree, :1955-1971 */
					uint64_t payload = chunk_tree_ll128(size, channels[c], log2_nnodes);
					if (payload > max_chunk || (payload == max_chunk && channels[c] > best)) {
						max_chunk = payload;
						best = channels[c];
					}
				}
				nchannels = best;
			}
			if (platform == OFI_AMD_PLATFORM_P6 && size <= 32 * 1024 * 1024 &&
			    algorithm == ALGO_PAT && protocol == PROTO_SIMPLE && nodes == ranks) {
				/* calculateBestNChannelPat, :1943-1953 */
				nchannels = 0;
				if (size <= nodes * 65536) nchannels = 1;
				else if (size <= nodes * 65536 * 2) nchannels = 2;
			}
		}
	}
	choice[idx * 4 + 0] = (int8_t)algorithm;
	choice[idx * 4 + 1] = (int8_t)protocol;
	*reinterpret_cast<int16_t *>(&choice[idx * 4 + 2]) = (int16_t)nchannels;
}

/* ---- host side: building the log2-space polygon tables ---- */

constexpr double kTunerMaxRanks = 1024.0 * 1024;                /* nccl_ofi_tuner_region.h:69 */
constexpr double kTunerMaxSize = 100.0 * 1024 * 1024 * 1024;   /* :74 */

/* transform_log2, include/tuner/nccl_ofi_tuner_region.h:87-109 */
pt_t to_log2(pt_t p)
{
	const double eps = 1e-6;
	if (p.x == 0) p.x = eps;
	if (p.y == 0) p.y = eps;
	return pt_t{ std::log2(p.x), std::log2(p.y) };
}

/* extend_region, src/tuner/nccl_ofi_regions.cpp:254-289 */
pt_t extend(pt_t a, pt_t b, pt_t z)
{
	a = to_log2(a);
	b = to_log2(b);
	z = to_log2(z);
	pt_t ret;
	if (a.x == b.x) {
		ret = pt_t{ a.x, z.y };
	} else if (a.y == b.y) {
		ret = pt_t{ z.x, a.y };
	} else {
		double m = (a.y - b.y) / (a.x - b.x);
		double c = b.y - m * b.x;
		double projected_zy = m * z.x + c;
		if (projected_zy < z.y) {
			ret = pt_t{ z.x, projected_zy };
		} else {
			ret = pt_t{ (z.y - c) / m, z.y };
		}
	}
	return pt_t{ std::pow(2.0, ret.x), std::pow(2.0, ret.y) };
}

template <typename T>
int upload(const std::vector<T> &host, T **dev)
{
	*dev = nullptr;
	if (host.empty()) {
		return 0;
	}
	OFI_AMD_HIP_TRY(hipMalloc((void **)dev, host.size() * sizeof(T)));
	OFI_AMD_HIP_TRY(hipMemcpy(*dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
	return 0;
}

} // namespace

struct ofi_amd_tuner_plan {
	grid_dims_t g;
	region_tables_t t;
	uint64_t points;
	uint64_t cells;
	/* owned device allocations */
	int32_t *d_colls, *d_algos, *d_poly;
	uint64_t *d_sizes, *d_nodes;
	uint32_t *d_ppn;
	double *d_log2_nodes, *d_log2_sizes, *d_log2_ranks;
	pt_t *d_verts;
	/* per-call variant / platform staging (device) */
	ofi_amd_tuner_variant_t *d_variants;
	int32_t *d_platforms;
	uint32_t variants_cap, platforms_cap;
};

using namespace ofi_amd;

extern "C" {

int ofi_amd_tuner_plan_destroy(ofi_amd_tuner_plan_t *plan)
{
	if (!plan) {
		return -EINVAL;
	}
	(void)hipFree(plan->d_colls);
	(void)hipFree(plan->d_algos);
	(void)hipFree(plan->d_poly);
	(void)hipFree(plan->d_sizes);
	(void)hipFree(plan->d_nodes);
	(void)hipFree(plan->d_ppn);
	(void)hipFree(plan->d_log2_nodes);
	(void)hipFree(plan->d_log2_sizes);
	(void)hipFree(plan->d_log2_ranks);
	(void)hipFree(plan->d_verts);
	(void)hipFree(plan->d_variants);
	(void)hipFree(plan->d_platforms);
	delete plan;
	return 0;
}

int ofi_amd_tuner_plan_create(const int32_t *colls, uint32_t n_colls, const uint64_t *sizes,
			      uint32_t n_sizes, const uint64_t *nodes, uint32_t n_nodes,
			      const uint32_t *ppn, uint32_t n_ppn, const int32_t *algos,
			      uint32_t n_algos, ofi_amd_tuner_plan_t **out)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!colls || !sizes || !nodes || !ppn || !algos || !out || n_colls == 0 || n_sizes == 0 ||
	    n_nodes == 0 || n_ppn == 0 || n_algos == 0) {
		return -EINVAL;
	}
	for (uint32_t i = 0; i < n_colls; i++) {
		if (colls[i] < 0 || colls[i] >= NUM_FUNCS) {
			return -EINVAL;
		}
	}
	for (uint32_t i = 0; i < n_algos; i++) {
		if (algos[i] < 0 || algos[i] >= NUM_ALGOS) {
			return -EINVAL;
		}
	}
	for (uint32_t i = 0; i < n_nodes; i++) {
		if (nodes[i] == 0 || nodes[i] > (1u << 30)) {
			return -EINVAL;
		}
	}
	for (uint32_t i = 0; i < n_ppn; i++) {
		if (ppn[i] == 0) {
			return -EINVAL;
		}
	}

	auto *plan = new (std::nothrow) ofi_amd_tuner_plan();
	if (!plan) {
		return -ENOMEM;
	}
	std::memset(plan, 0, sizeof(*plan));

	/* query coordinates, through the host's libm */
	std::vector<double> log2_nodes(n_nodes), log2_sizes(n_sizes), log2_ranks((size_t)n_nodes * n_ppn);
	for (uint32_t i = 0; i < n_nodes; i++) {
		log2_nodes[i] = std::log2((double)nodes[i]);
		for (uint32_t j = 0; j < n_ppn; j++) {
			log2_ranks[(size_t)i * n_ppn + j] = to_log2(pt_t{ 1.0, (double)(nodes[i] * ppn[j]) }).y;
		}
	}
	for (uint32_t i = 0; i < n_sizes; i++) {
		log2_sizes[i] = to_log2(pt_t{ (double)sizes[i], 1.0 }).x;
	}

	/* polygons: extension points, then set_regions' per-vertex log2 (:224-247) */
	std::vector<int32_t> poly;
	std::vector<pt_t> verts;
	region_tables_t &t = plan->t;
	for (int p = 0; p < kNumPlatforms; p++) {
		for (int s = 0; s < kNumShapes; s++) {
			for (int c = 0; c < NUM_FUNCS; c++) {
				t.set_first[p][s][c] = -1;
				t.set_count[p][s][c] = 0;
			}
		}
	}
	const pt_t z = { kTunerMaxSize, kTunerMaxRanks };
	for (int s = 0; s < OFI_REGION_NUM_SETS; s++) {
		const int *set = ofi_region_sets[s];
		const int shape = set[1] == 8 ? 0 : (set[1] == 2 ? 1 : 2);
		pt_t ext[8];
		for (int e = 0; e < set[6]; e++) {
			const double *r = ofi_region_exts[set[5] + e];
			ext[e] = extend(pt_t{ r[0], r[1] }, pt_t{ r[2], r[3] }, z);
		}
		t.set_first[set[0]][shape][set[2]] = (int32_t)(poly.size() / 4);
		t.set_count[set[0]][shape][set[2]] = set[4];
		for (int q = 0; q < set[4]; q++) {
			const int *pd = ofi_region_polys[set[3] + q];
			if (pd[3] > kMaxVertices) {
				delete plan;
				return -EINVAL;
			}
			poly.push_back(pd[0]);
			poly.push_back(pd[1]);
			poly.push_back((int32_t)verts.size());
			poly.push_back(pd[3]);
			for (int v = 0; v < pd[3]; v++) {
				const int *kind = ofi_region_vert_kind[pd[2] + v];
				const double *xy = ofi_region_vert_xy[pd[2] + v];
				pt_t pt;
				pt.x = kind[0] == 0 ? xy[0]
						    : (((kind[0] - 1) & 1) == 0 ? ext[(kind[0] - 1) / 2].x
										: ext[(kind[0] - 1) / 2].y);
				pt.y = kind[1] == 0 ? xy[1]
						    : (((kind[1] - 1) & 1) == 0 ? ext[(kind[1] - 1) / 2].x
										: ext[(kind[1] - 1) / 2].y);
				verts.push_back(to_log2(pt));
			}
		}
	}
	t.far_point = to_log2(pt_t{ 2.0 * kTunerMaxSize, 2.0 * kTunerMaxRanks });

	rc = upload(std::vector<int32_t>(colls, colls + n_colls), &plan->d_colls);
	if (rc == 0) rc = upload(std::vector<int32_t>(algos, algos + n_algos), &plan->d_algos);
	if (rc == 0) rc = upload(std::vector<uint64_t>(sizes, sizes + n_sizes), &plan->d_sizes);
	if (rc == 0) rc = upload(std::vector<uint64_t>(nodes, nodes + n_nodes), &plan->d_nodes);
	if (rc == 0) rc = upload(std::vector<uint32_t>(ppn, ppn + n_ppn), &plan->d_ppn);
	if (rc == 0) rc = upload(log2_nodes, &plan->d_log2_nodes);
	if (rc == 0) rc = upload(log2_sizes, &plan->d_log2_sizes);
	if (rc == 0) rc = upload(log2_ranks, &plan->d_log2_ranks);
	if (rc == 0) rc = upload(poly, &plan->d_poly);
	if (rc == 0) rc = upload(verts, &plan->d_verts);
	if (rc != 0) {
		ofi_amd_tuner_plan_destroy(plan);
		return rc;
	}

	grid_dims_t &g = plan->g;
	g.n_colls = n_colls;
	g.n_sizes = n_sizes;
	g.n_nodes = n_nodes;
	g.n_ppn = n_ppn;
	g.n_algos = n_algos;
	g.colls = plan->d_colls;
	g.sizes = plan->d_sizes;
	g.nodes = plan->d_nodes;
	g.ppn = plan->d_ppn;
	g.algos = plan->d_algos;
	g.log2_nodes = plan->d_log2_nodes;
	t.poly = plan->d_poly;
	t.verts = plan->d_verts;
	t.log2_sizes = plan->d_log2_sizes;
	t.log2_ranks = plan->d_log2_ranks;
	plan->points = (uint64_t)n_colls * n_sizes * n_nodes * n_ppn;
	plan->cells = plan->points * n_algos * NUM_PROTOS;
	*out = plan;
	return 0;
}

uint64_t ofi_amd_tuner_plan_points(const ofi_amd_tuner_plan_t *plan)
{
	return plan ? plan->points : 0;
}

uint64_t ofi_amd_tuner_plan_cells(const ofi_amd_tuner_plan_t *plan)
{
	return plan ? plan->cells : 0;
}

int ofi_amd_tuner_model_grid(ofi_amd_tuner_plan_t *plan, const ofi_amd_tuner_variant_t *variants,
			     uint32_t n_variants, double *d_cost, int8_t *d_choice, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!plan || !variants || n_variants == 0) {
		return -EINVAL;
	}
	for (uint32_t i = 0; i < n_variants; i++) {
		if (variants[i].platform < 0 || variants[i].platform >= kNumPlatforms) {
			return -EINVAL;
		}
	}
	hipStream_t s = as_stream(stream);
	if (n_variants > plan->variants_cap) {
		OFI_AMD_HIP_TRY(hipStreamSynchronize(s));
		(void)hipFree(plan->d_variants);
		plan->d_variants = nullptr;
		plan->variants_cap = 0;
		OFI_AMD_HIP_TRY(hipMalloc((void **)&plan->d_variants, sizeof(*variants) * n_variants));
		plan->variants_cap = n_variants;
	}
	OFI_AMD_HIP_TRY(hipMemcpyAsync(plan->d_variants, variants, sizeof(*variants) * n_variants,
				       hipMemcpyHostToDevice, s));
	if (d_cost) {
		const uint64_t total = plan->cells * n_variants;
		if (total > (1ull << 38)) {
			return -EINVAL;
		}
		hipLaunchKernelGGL(model_cost_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0,
				   s, plan->g, plan->d_variants, n_variants, plan->cells, d_cost);
	}
	if (d_choice) {
		const uint64_t total = plan->points * n_variants;
		hipLaunchKernelGGL(model_choice_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256),
				   0, s, plan->g, plan->d_variants, n_variants, plan->points, d_choice);
	}
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_tuner_region_grid(ofi_amd_tuner_plan_t *plan, const int32_t *platforms,
			      uint32_t n_platforms, int8_t *d_choice, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!plan || !platforms || n_platforms == 0 || !d_choice) {
		return -EINVAL;
	}
	for (uint32_t i = 0; i < n_platforms; i++) {
		if (platforms[i] < 0 || platforms[i] >= kNumPlatforms) {
			return -EINVAL;
		}
	}
	hipStream_t s = as_stream(stream);
	if (n_platforms > plan->platforms_cap) {
		OFI_AMD_HIP_TRY(hipStreamSynchronize(s));
		(void)hipFree(plan->d_platforms);
		plan->d_platforms = nullptr;
		plan->platforms_cap = 0;
		OFI_AMD_HIP_TRY(hipMalloc((void **)&plan->d_platforms, sizeof(int32_t) * n_platforms));
		plan->platforms_cap = n_platforms;
	}
	OFI_AMD_HIP_TRY(hipMemcpyAsync(plan->d_platforms, platforms, sizeof(int32_t) * n_platforms,
				       hipMemcpyHostToDevice, s));
	const uint64_t total = plan->points * n_platforms;
	hipLaunchKernelGGL(region_choice_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s,
			   plan->g, plan->t, plan->d_platforms, n_platforms, plan->points, d_choice);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

} /* extern "C" */
