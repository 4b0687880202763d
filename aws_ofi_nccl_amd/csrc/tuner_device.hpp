/*
 * Device functions of the tuner shared by the grid kernels (tuner_grid.hip) and the
 * point-query kernel (tuner_query.hip).
 *
 * Model: nccl_ofi_tuner_compute_cost and model_get_coll_info_internal_v3 / _v2,
 * src/tuner/nccl_ofi_model.cpp:13-309.  The reference computes in fp32 with two
 * double sub-expressions (log2 of the node count) and never fuses a multiply with
 * an add; every rounding step is kept (explicit round-to-nearest intrinsics, files
 * built with contraction off) and log2(nodes) arrives precomputed by the host's
 * libm, so costs match bit for bit.
 *
 * Regions: region_get_coll_info_internal_v3 / _v2, src/tuner/nccl_ofi_regions.cpp:
 * 1995-2157, with is_inside_region (:159-221) and the channel / chunk heuristics
 * (:1883-1971, :2159-2306).  Polygons and query coordinates arrive log2-transformed
 * from the host.  The reference's `long double` intermediates (:91, :50-56) are
 * 80-bit on x86-64 and plain double here; that can only move a point that lies
 * within ~1e-16 of the 1e-10 on-edge threshold.
 */
#ifndef OFI_AMD_TUNER_DEVICE_HPP_
#define OFI_AMD_TUNER_DEVICE_HPP_

#include <cmath>
#include <cstdint>

#include <hip/hip_runtime.h>

#include "ofi_amd_hotpath.h"

namespace ofi_amd_tuner {

/* nccl/tuner.h:14-41 */
enum { FUNC_ALLGATHER = 2, FUNC_REDUCESCATTER = 3, FUNC_ALLREDUCE = 4, NUM_FUNCS = 5 };
enum { ALGO_TREE = 0, ALGO_RING = 1, ALGO_COLLNET_DIRECT = 2, ALGO_COLLNET_CHAIN = 3,
       ALGO_NVLS = 4, ALGO_NVLS_TREE = 5, ALGO_PAT = 6, NUM_ALGOS = 7 };
enum { PROTO_LL = 0, PROTO_LL128 = 1, PROTO_SIMPLE = 2, NUM_PROTOS = 3 };

constexpr int kNumPlatforms = 4;
constexpr int kNumShapes = 3; /* ranks == 8*nodes, 2*nodes, nodes */
constexpr int kMaxVertices = 20;
constexpr uint32_t kAllAllowed = (1u << (NUM_ALGOS * NUM_PROTOS)) - 1;

__host__ __device__ inline bool allowed(uint32_t mask, int algo, int proto)
{
	return (mask >> (algo * NUM_PROTOS + proto)) & 1u;
}

struct model_params_t {
	float net_lat;
	float internode_bw;
	float intranode_bw;
	int num_rails;
};

/* src/tuner/nccl_ofi_model.cpp:13-44; the bandwidths are double constant
 * expressions narrowed to float once, as there. */
__device__ __forceinline__ model_params_t model_params(int platform)
{
	if (platform == OFI_AMD_PLATFORM_P5EN) {
		return model_params_t{ 18.0f, (float)(25.0 * 1024 * 1024 * 1024 * 1e-6),
				       (float)(20.0 * 1024 * 1024 * 1024 * 1e-6), 2 };
	}
	return model_params_t{ 20.0f, (float)(12.5 * 1024 * 1024 * 1024 * 1e-6),
			       (float)(20.0 * 1024 * 1024 * 1024 * 1e-6), 4 };
}

/* nccl_nvlink_lat, the same table for both modelled platforms (:19-27, :34-42) */
__device__ __forceinline__ float nvlink_lat(int algo, int proto)
{
	switch (algo * NUM_PROTOS + proto) {
	case ALGO_TREE * 3 + PROTO_LL: return .6f;
	case ALGO_TREE * 3 + PROTO_LL128: return 1.25f;
	case ALGO_TREE * 3 + PROTO_SIMPLE: return 28.f;
	case ALGO_RING * 3 + PROTO_LL: return .6f;
	case ALGO_RING * 3 + PROTO_LL128: return 1.9f;
	case ALGO_RING * 3 + PROTO_SIMPLE: return 3.4f;
	case ALGO_COLLNET_DIRECT * 3 + PROTO_SIMPLE: return 3.7f;
	case ALGO_COLLNET_CHAIN * 3 + PROTO_SIMPLE: return 2.8f;
	case ALGO_NVLS * 3 + PROTO_SIMPLE: return 23.f;
	case ALGO_NVLS_TREE * 3 + PROTO_SIMPLE: return 23.f;
	default: return 0.f;
	}
}

__host__ __device__ inline bool platform_has_model(int platform)
{
	return platform == OFI_AMD_PLATFORM_P5_P5E || platform == OFI_AMD_PLATFORM_P5EN;
}

/* nccl_ofi_tuner_compute_cost, src/tuner/nccl_ofi_model.cpp:46-122 */
__device__ inline float model_cost(int platform, int coll, int algo, int proto, int pipe_ops,
				   uint64_t size, uint64_t num_ranks, uint64_t num_nodes,
				   double log2_nodes, int num_channels, int net_comp_overhead)
{
	if (coll != FUNC_ALLREDUCE) {
		return -1.0f;
	}
	const model_params_t params = model_params(platform);
	const float net_lat = (proto == PROTO_SIMPLE)
				      ? __fadd_rn(params.net_lat, (float)net_comp_overhead)
				      : params.net_lat;
	const float p2p_lat = nvlink_lat(algo, proto);
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

/* The three protocols of one algorithm at once: cell for cell the operations of model_cost above,
 * in the same order, with what the three cells share worked out once (the step counts and their
 * conversions, the base bandwidth, the rank quotient and the log term).  size_f = (float)size,
 * ranks_over_nodes = num_ranks / num_nodes (a grid knows it without dividing). */
__device__ inline void model_cost_protos(int platform, int coll, int algo, int pipe_ops, float size_f,
					 uint64_t num_ranks, uint64_t num_nodes, uint64_t ranks_over_nodes,
					 double log2_nodes, int num_channels, int net_comp_overhead,
					 float out[NUM_PROTOS])
{
	out[PROTO_LL] = out[PROTO_LL128] = out[PROTO_SIMPLE] = -1.0f;
	if (coll != FUNC_ALLREDUCE || (algo != ALGO_RING && algo != ALGO_TREE && algo != ALGO_NVLS_TREE)) {
		return;
	}
	const model_params_t params = model_params(platform);
	const float net_lat_of[NUM_PROTOS] = { params.net_lat, params.net_lat,
					       __fadd_rn(params.net_lat, (float)net_comp_overhead) };
	const float rails_bw = __fmul_rn(params.internode_bw, (float)params.num_rails);
	float latency[NUM_PROTOS], bw;
	if (algo == ALGO_RING) {
		const int num_steps = (int)(2 * (num_ranks - 1));
		const int num_internode_steps = (int)(2 * num_nodes);
		const float inter = (float)num_internode_steps, rest = (float)(num_steps - num_internode_steps);
#pragma unroll
		for (int proto = 0; proto < NUM_PROTOS; proto++) {
			latency[proto] = __fadd_rn(__fmul_rn(inter, net_lat_of[proto]),
						   __fmul_rn(rest, nvlink_lat(ALGO_RING, proto)));
		}
		bw = __fmul_rn(rails_bw, (float)num_channels);
	} else if (algo == ALGO_NVLS_TREE) {
#pragma unroll
		for (int proto = 0; proto < NUM_PROTOS; proto++) {
			const double t = __dadd_rn((double)nvlink_lat(ALGO_NVLS_TREE, proto),
						   __dmul_rn(log2_nodes, (double)net_lat_of[proto]));
			latency[proto] = (float)__dmul_rn(2.0, t);
		}
		const float half = __fdiv_rn(rails_bw, 2.0f);
		bw = __fmul_rn(half < params.intranode_bw ? half : params.intranode_bw, (float)num_channels);
	} else {
		const float hops = (float)(2 * (ranks_over_nodes - 1));
		const double log_term = __dmul_rn(2.0, log2_nodes);
#pragma unroll
		for (int proto = 0; proto < NUM_PROTOS; proto++) {
			const float a = __fmul_rn(hops, nvlink_lat(ALGO_TREE, proto));
			const double b = __dmul_rn(log_term, (double)net_lat_of[proto]);
			latency[proto] = (float)__dadd_rn((double)a, b);
		}
		bw = __fdiv_rn(__fmul_rn(rails_bw, (float)num_channels), 2.0f);
	}
	const float bw_of[NUM_PROTOS] = { (float)__dmul_rn((double)bw, 0.5), (float)__dmul_rn((double)bw, 0.9375), bw };
	const float pipe = (float)pipe_ops;
#pragma unroll
	for (int proto = 0; proto < NUM_PROTOS; proto++) {
		out[proto] = __fadd_rn(__fmul_rn(latency[proto], pipe), __fdiv_rn(size_f, bw_of[proto]));
	}
}

/* model_get_coll_info_internal_v3 (:154-234); with the NVLS-tree bit of `mask`
 * clear it is _v2 with nvlsSupport == 0 (:236-309).  The model never looks at
 * NCCL's cost table, so no other bit of the mask matters here.  cost_of(algo, proto) is the
 * cell's cost, negative when not modelled. */
template <typename F>
__device__ __forceinline__ void model_choose_with(int platform, int coll, uint64_t size, uint64_t ranks,
						  uint64_t nodes, uint32_t mask, F cost_of, int &chosen_algo,
						  int &chosen_proto)
{
	chosen_algo = -1;
	chosen_proto = -1;
	if (!platform_has_model(platform) || nodes <= 2) { /* :178 */
		return;
	}
	const bool nvls = allowed(mask, ALGO_NVLS_TREE, PROTO_SIMPLE);
	if (platform == OFI_AMD_PLATFORM_P5_P5E && coll == FUNC_ALLREDUCE && nodes == 16 &&
	    ranks == 128 && nvls && size > 3ULL * 1024 * 1024 * 1024 &&
	    size <= 5ULL * 1024 * 1024 * 1024) { /* :183-192 */
		chosen_algo = ALGO_NVLS_TREE;
		chosen_proto = PROTO_SIMPLE;
		return;
	}
	float lowest = 3.402823466e+38f; /* FLT_MAX */
	for (int algo = 0; algo < NUM_ALGOS; algo++) {
		if (algo == ALGO_COLLNET_DIRECT || algo == ALGO_COLLNET_CHAIN || algo == ALGO_NVLS) {
			continue;
		}
		if (algo == ALGO_NVLS_TREE && !nvls) {
			continue;
		}
		for (int proto = 0; proto < NUM_PROTOS; proto++) {
			if (algo == ALGO_NVLS_TREE && proto != PROTO_SIMPLE) {
				continue;
			}
			float c = cost_of(algo, proto);
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

__device__ inline void model_choose(int platform, int coll, uint64_t size, uint64_t ranks,
				    uint64_t nodes, double log2_nodes, int pipe_ops, int num_channels,
				    int net_comp_overhead, uint32_t mask, int &chosen_algo,
				    int &chosen_proto)
{
	model_choose_with(
		platform, coll, size, ranks, nodes, mask,
		[&](int algo, int proto) -> float {
			return model_cost(platform, coll, algo, proto, pipe_ops, size, ranks, nodes, log2_nodes,
					  num_channels, net_comp_overhead);
		},
		chosen_algo, chosen_proto);
}

/* ------------------------------------------------------------------ regions */

struct pt_t {
	double x, y;
};

struct region_tables_t {
	/* [platform][shape][coll] -> first polygon / count (0 when no regions) */
	int32_t set_first[kNumPlatforms][kNumShapes][NUM_FUNCS];
	int32_t set_count[kNumPlatforms][kNumShapes][NUM_FUNCS];
	const int32_t *poly; /* per polygon {algo, proto, first_vertex, num_vertices} */
	const pt_t *verts;   /* log2 space */
	const double *bbox;  /* per polygon {min_x, max_x, min_y, max_y} as is_inside_region finds them */
	pt_t far_point;      /* log2 of (2*max size, 2*max ranks) */
};

__device__ __forceinline__ pt_t vsub(pt_t a, pt_t b) { return pt_t{ a.x - b.x, a.y - b.y }; }
__device__ __forceinline__ double vdot(pt_t a, pt_t b) { return a.x * b.x + a.y * b.y; }
__device__ __forceinline__ double vcross(pt_t a, pt_t b) { return a.x * b.y - a.y * b.x; }

/* intersect, src/tuner/nccl_ofi_regions.cpp:77-109 */
__device__ inline int intersect(pt_t x0, pt_t x1, pt_t y0, pt_t y1, double eps, pt_t *sect)
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
__device__ inline double seg_distance(pt_t x, pt_t y0, pt_t y1, double eps)
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

/*
 * Certain-answer forms of the two per-edge tests.  Each evaluates the quotient of `intersect`
 * with an approximate reciprocal (hardware estimate plus one Newton step: relative error below
 * 1e-12 against the 1e-5 margins used here) and says whether the exact code's answer is already
 * certain from it.  They are straight-line code -- no branch, no division, no square root -- so
 * the walk over a polygon's edges can overlap the arithmetic of several edges; a point for which
 * any edge is not certain (a quotient near one of the thresholds, a degenerate edge, a foot point
 * close to the edge) is run again through the exact code above, so results are the exact code's.
 */
__device__ __forceinline__ double approx_rcp(double d)
{
	double r = __builtin_amdgcn_rcp(d);
	return r * (2.0 - d * r);
}

/* |a - t| far beyond what the approximate quotient can be off by */
__device__ __forceinline__ bool clear_of(double a, double t)
{
	return fabs(a - t) > 1e-5 * (1.0 + fabs(a));
}

/* Whether intersect(x0, x0 + dx, y0, y1, eps, nullptr) == 1; `certain` is cleared when only the
 * exact quotient can tell. */
__device__ __forceinline__ bool crosses_edge(pt_t x0, pt_t dx, pt_t y0, pt_t y1, double eps, bool &certain)
{
	const pt_t dy = vsub(y1, y0);
	const double d = vcross(dy, dx);
	const bool parallel = fabs(d) < eps; /* the exact code answers 0 */
	const double r = approx_rcp(parallel ? 1.0 : d);
	const double a = (vcross(x0, dx) - vcross(y0, dx)) * r;
	const double b = (vcross(x0, dy) - vcross(y0, dy)) * r;
	const bool a_clear = clear_of(a, 0.0) && clear_of(a, 1.0);
	const bool b_clear = clear_of(b, 0.0) && clear_of(b, 1.0);
	const bool a_in = a > 0.0 && a < 1.0; /* with a_clear: inside (eps, 1 - eps); else beyond -eps or 1 + eps */
	const bool b_in = b > 0.0 && b < 1.0;
	certain &= parallel | (a_clear & (!a_in | b_clear));
	return !parallel && a_in && b_in;
}

/* false only when seg_distance(x, y0, y1, eps) is certainly not below eps */
__device__ __forceinline__ bool may_touch_edge(pt_t x, pt_t y0, pt_t y1, double eps)
{
	const pt_t dy = vsub(y1, y0);
	pt_t x1;
	x1.x = x.x + dy.y;
	x1.y = x.y - dy.x;
	const pt_t dx = vsub(x1, x);
	const double d = vcross(dy, dx);
	const bool degenerate = fabs(d) < eps; /* the exact code leaves the foot point unset here */
	const double a = (vcross(x, dx) - vcross(y0, dx)) * approx_rcp(degenerate ? 1.0 : d);
	const pt_t s = { y0.x + a * dy.x - x.x, y0.y + a * dy.y - x.y };
	/* the foot point computed exactly differs from this one by ~1e-12 (1 + |a|)(1 + |dy|) at most */
	const double far = 1e-4 * (1.0 + fabs(a)) * (1.0 + fabs(dy.x) + fabs(dy.y));
	return degenerate || !(vdot(s, s) > far * far);
}

/* The bounds is_inside_region computes (:177-196): selections only, so the host can do it
 * once per polygon with the same result.  The y bounds start from vertex 1 as in the reference
 * (:177-178). */
__host__ __device__ inline void region_bounds(const pt_t *v, int n, double out[4])
{
	double min_x = v[0].x, max_x = v[0].x, min_y = v[1].y, max_y = v[1].y;
	for (int i = 0; i < n; i++) {
		if (v[i].x > max_x) max_x = v[i].x;
		if (v[i].x < min_x) min_x = v[i].x;
		if (v[i].y > max_y) max_y = v[i].y;
		if (v[i].y < min_y) min_y = v[i].y;
	}
	out[0] = min_x;
	out[1] = max_x;
	out[2] = min_y;
	out[3] = max_y;
}

/* is_inside_region, :159-221; `bounds` is region_bounds of the same polygon */
__device__ __forceinline__ int inside_region(pt_t point, const pt_t *v, int n, const double *bounds,
					      pt_t far_point)
{
	const double eps = 1e-10;
	const double min_x = bounds[0], max_x = bounds[1], min_y = bounds[2], max_y = bounds[3];
	/* The reference looks for a point on an edge first (result 0) and rejects by bounding
	 * box second (result -1).  A point more than 1e-6 outside the box cannot be within
	 * 1e-10 of an edge -- edges lie inside the box, and the foot of the perpendicular may
	 * leave the segment by at most eps times its length -- so for such a point the second
	 * answer is known without looking at the edges.  Most polygons are dismissed here. */
	const double margin = 1e-6;
	if (point.x < min_x - margin || point.x > max_x + margin || point.y < min_y - margin ||
	    point.y > max_y + margin) {
		return -1;
	}
	/* One branch-free walk over the edges (at most 20, one bit each) serves both of the
	 * reference's loops, the on-edge search (:168-175) and the crossing count (:207-219); the
	 * edges whose answer it could not be certain of are then put through the exact code. */
	const pt_t ray = vsub(far_point, point);
	uint32_t touch = 0, unsure = 0;
	int crosses = 0;
	pt_t a = v[n - 1];
#pragma unroll 4
	for (int i = 0; i < n; i++) { /* edge (i - 1, i): the same edges, starting from the closing one */
		const pt_t b = v[i];
		bool certain = true;
		const bool crossing = crosses_edge(point, ray, a, b, eps, certain);
		touch |= (uint32_t)may_touch_edge(point, a, b, eps) << i;
		unsure |= (uint32_t)!certain << i;
		crosses += (crossing & certain) ? 1 : 0;
		a = b;
	}
	while (touch != 0) {
		const int i = __ffs(touch) - 1;
		touch &= touch - 1;
		if (seg_distance(point, v[i == 0 ? n - 1 : i - 1], v[i], eps) < eps) {
			return 0;
		}
	}
	if (point.x < min_x || point.x > max_x || point.y < min_y || point.y > max_y) {
		return -1;
	}
	while (unsure != 0) {
		const int i = __ffs(unsure) - 1;
		unsure &= unsure - 1;
		if (intersect(point, far_point, v[i == 0 ? n - 1 : i - 1], v[i], eps, nullptr) == 1) {
			crosses++;
		}
	}
	return (crosses & 1) ? 1 : -1;
}

/* calculateChunkSizeTreeLL128, :1883-1938 (constants: include/internal/tuner/nccl_defaults.h) */
__device__ inline uint64_t chunk_tree_ll128(uint64_t message_size, int nChannels, int log2_nnodes)
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

__device__ __forceinline__ int log2i_nodes(uint64_t nodes)
{
	const int x = (int)nodes; /* log2i(int), include/internal/tuner/nccl_defaults.h:92-104 */
	return x <= 0 ? -1 : 31 - __clz(x);
}

/* Which polygon set answers for (platform, collective, ranks per node): shape selection as in
 * the per-platform init functions (:302,:485,:675,:768,:878,...).  count 0: no regions. */
__host__ __device__ __forceinline__ void region_set(const region_tables_t &t, int platform, int coll, uint64_t ranks,
					    uint64_t nodes, int &first, int &count)
{
	first = 0;
	count = 0;
	int shape = -1;
	if (ranks == 8 * nodes) shape = 0;
	else if (ranks == 2 * nodes && platform == OFI_AMD_PLATFORM_P5_P5E) shape = 1;
	else if (ranks == nodes) shape = 2;
	if (platform < 0 || platform >= kNumPlatforms || shape < 0 || coll < 0 || coll >= NUM_FUNCS ||
	    t.set_count[platform][shape][coll] <= 0) {
		return;
	}
	first = t.set_first[platform][shape][coll];
	count = t.set_count[platform][shape][coll];
}

/* The loop of region_get_coll_info_internal_v3 (:2106-2128) over one set: the first polygon that
 * holds the point (inside or on an edge) wins.  Regions whose (algo, proto) bit is clear in
 * `mask` are passed over: for v3 those are the cells NCCL marked -1 or that lie beyond numAlgo /
 * numProto (:2109-2114); for v2 PAT and, without NVLS support, NVLS tree (:2023-2030).
 * poly: 4 ints per polygon, its vertex index relative to `verts`; bounds: 4 doubles per polygon.
 * The arrays may live in global memory or in LDS. */
__device__ __forceinline__ int region_pick(const int32_t *poly, const double *bounds, const pt_t *verts,
					    int count, pt_t p, uint32_t mask, pt_t far_point, int &a, int &pr)
{
	int in_out = -1;
	a = -1;
	pr = -1;
	for (int i = 0; i < count && in_out < 0; i++) {
		a = poly[i * 4 + 0];
		pr = poly[i * 4 + 1];
		if (!allowed(mask, a, pr)) {
			continue;
		}
		in_out = inside_region(p, &verts[poly[i * 4 + 2]], poly[i * 4 + 3], &bounds[i * 4], far_point);
	}
	return in_out;
}

/* The nChannels override of the chosen region (:2135-2153), -1 when there is none. */
__device__ __forceinline__ int region_channels(int platform, uint64_t size, uint64_t ranks, uint64_t nodes,
						int algorithm, int protocol)
{
	int nchannels = -1;
	if (platform == OFI_AMD_PLATFORM_P6 && size >= 4 * 1024 * 1024 && size <= 32 * 1024 * 1024 &&
	    algorithm == ALGO_TREE && protocol == PROTO_LL128 && nodes * 8 == ranks) { /* :2140-2146 */
		const int log2_nnodes = log2i_nodes(nodes);
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
	if (platform == OFI_AMD_PLATFORM_P6 && size <= 32 * 1024 * 1024 && algorithm == ALGO_PAT &&
	    protocol == PROTO_SIMPLE && nodes == ranks) {
		/* calculateBestNChannelPat, :1943-1953 */
		nchannels = 0;
		if (size <= nodes * 65536) nchannels = 1;
		else if (size <= nodes * 65536 * 2) nchannels = 2;
	}
	return nchannels;
}

/* region_get_coll_info_internal_v3, :2070-2157, for one point with the tables in global memory.
 * p = (log2 bytes, log2 ranks) as transform_log2 gives them. */
__device__ inline void region_choose(const region_tables_t &t, int platform, int coll, uint64_t size,
				     uint64_t ranks, uint64_t nodes, pt_t p, uint32_t mask,
				     int &algorithm, int &protocol, int &nchannels)
{
	algorithm = -1;
	protocol = -1;
	nchannels = -1;
	int first, count;
	region_set(t, platform, coll, ranks, nodes, first, count);
	if (count <= 0 || nodes <= 2) {
		return;
	}
	int a, pr;
	if (region_pick(&t.poly[first * 4], &t.bbox[first * 4], t.verts, count, p, mask, t.far_point, a, pr) < 0) {
		return;
	}
	algorithm = a;
	protocol = pr;
	nchannels = region_channels(platform, size, ranks, nodes, a, pr);
}

/* region_get_chunk_size_internal, :2276-2306, with chunkSizeTuningTreeLL128P5en
 * (:2211-2274) and chunkSizeTuningAllGatherPatSimpleP5en (:2159-2209).
 * Returns 0 when the tuner leaves the chunk size alone. */
__device__ inline uint64_t region_chunk_size(int platform, int coll, uint64_t nbytes, int algo, int proto,
					     uint64_t ranks, uint64_t nodes)
{
	if (nodes != ranks || platform != OFI_AMD_PLATFORM_P5EN) {
		return 0;
	}
	if (coll == FUNC_ALLREDUCE && algo == ALGO_TREE && proto == PROTO_LL128) {
		const uint64_t nsteps = (uint64_t)(1 + log2i_nodes(nodes));
		uint64_t tuned = 288000;
		if (nbytes / tuned < 2 * nsteps * nsteps) tuned /= 2;
		if (nbytes / tuned < (uint64_t)(1.5 * (double)nsteps)) tuned /= 2;
		while (nbytes / tuned < nsteps + 1 && tuned > 18000) tuned /= 2;
		return tuned;
	}
	if (coll == FUNC_ALLGATHER && algo == ALGO_PAT && proto == PROTO_SIMPLE) {
		const uint64_t sat = nodes >= 16 ? 524288 : 1048576;
		const uint64_t T1 = nodes >= 16 ? 32 : (nodes < 8 ? nodes : 8) + 1;
		const uint64_t T2 = nodes < 16 ? nodes : 16;
		const uint64_t T3 = nodes < 8 ? nodes : 8;
		uint64_t tuned = sat;
		while (nbytes / tuned < T1 && tuned > sat / 2) tuned /= 2;
		while (nbytes / tuned < T2 && tuned > 65536) tuned /= 2;
		while (nbytes / tuned < T3 && tuned > 32768) tuned /= 2;
		return tuned;
	}
	return 0;
}

/* Host side (tuner_grid.hip): the process-wide device copy of the polygon tables and
 * transform_log2 (include/tuner/nccl_ofi_tuner_region.h:87-109) of one coordinate. */
int device_region_tables(region_tables_t *out);
double log2_coord(double v);

} // namespace ofi_amd_tuner

#endif
