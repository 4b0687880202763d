/*
 * CPU oracle (test infrastructure): tuner cost model and region tuner.
 *
 * Model: src/tuner/nccl_ofi_model.cpp:13-234.  Regions:
 * src/tuner/nccl_ofi_regions.cpp:32-289 (geometry), :1883-1971 and :2159-2306
 * (channel / chunk heuristics), :2070-2157 (decision), with
 * include/tuner/nccl_ofi_tuner_region.h:64-109.
 *
 * Build with -ffp-contract=off and without -ffast-math: the reference is
 * compiled for baseline x86-64, where no multiply-add is fused, and `long
 * double` is the 80-bit x87 type.
 */
#include <float.h>
#include <math.h>
#include <string.h>

#include "oracle.h"
#include "../aws_ofi_nccl_amd/csrc/region_tables.inc"

/* nccl/tuner.h:14-41 */
enum { FUNC_ALLGATHER = 2, FUNC_REDUCESCATTER = 3, FUNC_ALLREDUCE = 4 };
enum { ALGO_TREE = 0, ALGO_RING = 1, ALGO_COLLNET_DIRECT = 2, ALGO_COLLNET_CHAIN = 3,
       ALGO_NVLS = 4, ALGO_NVLS_TREE = 5, ALGO_PAT = 6, NUM_ALGOS = 7 };
enum { PROTO_LL = 0, PROTO_LL128 = 1, PROTO_SIMPLE = 2, NUM_PROTOS = 3 };

/* ------------------------------------------------------------------ model */

typedef struct {
	float net_lat;
	float internode_bw;
	float intranode_bw;
	int num_rails;
	float nvlink_lat[NUM_ALGOS][NUM_PROTOS];
} model_params_t;

/* src/tuner/nccl_ofi_model.cpp:13-44 */
static const model_params_t model_params[2] = {
	{
		.net_lat = 20.0,
		.internode_bw = (12.5 * 1024 * 1024 * 1024 * 1e-6),
		.intranode_bw = (20.0 * 1024 * 1024 * 1024 * 1e-6),
		.num_rails = 4,
		.nvlink_lat = { { .6, 1.25, 28 }, { .6, 1.9, 3.4 }, { 0, 0, 3.7 }, { 0, 0, 2.8 },
				{ 0, 0, 23 }, { 0, 0, 23 }, { 0, 0, 0 } },
	},
	{
		.net_lat = 18.0,
		.internode_bw = (25.0 * 1024 * 1024 * 1024 * 1e-6),
		.intranode_bw = (20.0 * 1024 * 1024 * 1024 * 1e-6),
		.num_rails = 2,
		.nvlink_lat = { { .6, 1.25, 28 }, { .6, 1.9, 3.4 }, { 0, 0, 3.7 }, { 0, 0, 2.8 },
				{ 0, 0, 23 }, { 0, 0, 23 }, { 0, 0, 0 } },
	},
};

/* nccl_ofi_tuner_compute_cost, :46-122.  Types are kept as in the reference:
 * float locals, int step counts, size_t dims; log2() of an integer is double. */
float oracle_model_cost(int platform, int coll, int algo, int proto, int pipe_ops,
			uint64_t size, uint64_t num_ranks, uint64_t num_nodes,
			int num_channels, int net_comp_overhead)
{
	const model_params_t *params = &model_params[platform];
	float cost = -1;
	float latency = 0;
	float bw = 0;
	float p2p_lat = 0;
	float net_lat = 0;
	int num_steps = 0;
	int num_internode_steps = 0;

	net_lat = (proto == PROTO_SIMPLE) ? params->net_lat + net_comp_overhead : params->net_lat;
	p2p_lat = params->nvlink_lat[algo][proto];

	if (coll != FUNC_ALLREDUCE) {
		return -1;
	}
	switch (algo) {
	case ALGO_RING:
		num_steps = 2 * (num_ranks - 1);
		num_internode_steps = 2 * num_nodes;
		latency = (num_internode_steps * net_lat)
			  + (num_steps - num_internode_steps) * p2p_lat;
		bw = params->internode_bw * params->num_rails * num_channels;
		break;
	case ALGO_NVLS_TREE: {
		float half = (params->internode_bw * params->num_rails) / 2;
		latency = 2 * (p2p_lat + (log2((double)num_nodes) * net_lat));
		/* std::min(a, b) yields b only when b < a */
		bw = (half < params->intranode_bw ? half : params->intranode_bw) * num_channels;
		break;
	}
	case ALGO_TREE:
		latency = ((2 * ((num_ranks / num_nodes) - 1) * p2p_lat)
			   + (2 * log2((double)num_nodes) * net_lat));
		bw = (params->internode_bw * params->num_rails * num_channels) / 2;
		break;
	default:
		return -1;
	}

	if (proto == PROTO_LL) {
		bw *= 0.5;
	} else if (proto == PROTO_LL128) {
		bw *= 0.9375;
	}

	cost = (latency * pipe_ops) + size / bw;
	return cost;
}

/* model_get_coll_info_internal_v3, :154-234 */
void oracle_model_decide(int platform, int coll, int pipe_ops, uint64_t size,
			 uint64_t num_ranks, uint64_t num_nodes, int num_channels,
			 int net_comp_overhead, int *algo_out, int *proto_out)
{
	oracle_model_decide_v2(platform, coll, pipe_ops, size, num_ranks, num_nodes, num_channels,
			       net_comp_overhead, 1, algo_out, proto_out);
}

/* model_get_coll_info_internal_v2, :236-309: as v3, but NVLS tree (and the P5 quirk
 * that selects it) only when NCCL reports NVLS support. */
void oracle_model_decide_v2(int platform, int coll, int pipe_ops, uint64_t size,
			    uint64_t num_ranks, uint64_t num_nodes, int num_channels,
			    int net_comp_overhead, int nvls_support, int *algo_out, int *proto_out)
{
	float lowest = FLT_MAX;
	int chosen_algo = -1, chosen_proto = -1;

	*algo_out = -1;
	*proto_out = -1;
	if (num_nodes <= 2) { /* :178 */
		return;
	}
	if (platform == ORACLE_PLAT_P5_P5E) { /* :183-192 */
		if (coll == FUNC_ALLREDUCE && num_nodes == 16 && num_ranks == 128 && nvls_support &&
		    size > 3ULL * 1024ULL * 1024ULL * 1024ULL &&
		    size <= 5ULL * 1024ULL * 1024ULL * 1024ULL) {
			*algo_out = ALGO_NVLS_TREE;
			*proto_out = PROTO_SIMPLE;
			return;
		}
	}
	for (int algo = 0; algo < NUM_ALGOS; algo++) {
		if (algo == ALGO_COLLNET_DIRECT || algo == ALGO_COLLNET_CHAIN || algo == ALGO_NVLS) {
			continue;
		}
		if (!nvls_support && algo == ALGO_NVLS_TREE) { /* :279-280 */
			continue;
		}
		for (int proto = 0; proto < NUM_PROTOS; proto++) {
			if (algo == ALGO_NVLS_TREE && proto != PROTO_SIMPLE) {
				continue;
			}
			float cost = oracle_model_cost(platform, coll, algo, proto, pipe_ops, size,
						       num_ranks, num_nodes, num_channels,
						       net_comp_overhead);
			if (cost < 0) {
				continue;
			}
			if (cost < lowest) {
				chosen_algo = algo;
				chosen_proto = proto;
				lowest = cost;
			}
		}
	}
	/* The reference writes table[chosen_algo][chosen_proto] even when both are
	 * -1 (:228-229); that out-of-bounds store is not reproduced: (-1,-1) means
	 * "no choice". */
	*algo_out = chosen_algo;
	*proto_out = chosen_proto;
}

/* --------------------------------------------------------------- regions */

#define MAX_VERTICES 20
#define TUNER_MAX_RANKS (1024.0 * 1024)
#define TUNER_MAX_SIZE (100.0 * 1024 * 1024 * 1024)

/* transform_log2, include/tuner/nccl_ofi_tuner_region.h:87-109 */
oracle_point_t oracle_region_log2(oracle_point_t p)
{
	const double eps = 1e-6;
	if (p.x == 0) {
		p.x = eps;
	}
	if (p.y == 0) {
		p.y = eps;
	}
	p.x = log2(p.x);
	p.y = log2(p.y);
	return p;
}

/* transform_pow2, :111-120 */
static oracle_point_t point_pow2(oracle_point_t p)
{
	p.x = pow(2.0, p.x);
	p.y = pow(2.0, p.y);
	return p;
}

static oracle_point_t vsub(oracle_point_t a, oracle_point_t b)
{
	oracle_point_t r = { a.x - b.x, a.y - b.y };
	return r;
}
static double vdot(oracle_point_t a, oracle_point_t b) { return a.x * b.x + a.y * b.y; }
static double vcross(oracle_point_t a, oracle_point_t b) { return a.x * b.y - a.y * b.x; }
/* a + s*b with s and the multiply-add in long double, src/tuner/nccl_ofi_regions.cpp:50-56 */
static oracle_point_t vmadd(oracle_point_t a, long double s, oracle_point_t b)
{
	oracle_point_t c;
	c.x = a.x + s * b.x;
	c.y = a.y + s * b.y;
	return c;
}

/* intersect, :77-109 */
static int intersect(oracle_point_t x0, oracle_point_t x1, oracle_point_t y0, oracle_point_t y1,
		     double eps, oracle_point_t *sect)
{
	oracle_point_t dx = vsub(x1, x0);
	oracle_point_t dy = vsub(y1, y0);
	double d = vcross(dy, dx);
	if (fabs(d) < eps) {
		return 0;
	}
	long double a = (long double)(vcross(x0, dx) - vcross(y0, dx)) / d;
	if (sect) {
		*sect = vmadd(y0, a, dy);
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
static double distance(oracle_point_t x, oracle_point_t y0, oracle_point_t y1, double eps)
{
	oracle_point_t dy = vsub(y1, y0);
	oracle_point_t x1, s = { 0, 0 };
	int r;

	x1.x = x.x + dy.y;
	x1.y = x.y - dy.x;
	r = intersect(x, x1, y0, y1, eps, &s);
	if (r == -1) {
		return HUGE_VAL;
	}
	s = vsub(s, x);
	return sqrt(vdot(s, s));
}

/* is_inside_region, :159-221 */
int oracle_region_inside(oracle_point_t point, const oracle_point_t *v, size_t n)
{
	size_t i, k;
	double min_x, max_x, min_y, max_y;
	const double eps = 1e-10;

	for (i = 0; i < n; i++) {
		k = (i + 1) % n;
		min_x = distance(point, v[i], v[k], eps);
		if (min_x < eps) {
			return 0;
		}
	}
	/* sic: y bounds start from vertex 1 (:177-178) */
	min_x = max_x = v[0].x;
	min_y = max_y = v[1].y;
	for (i = 0; i < n; i++) {
		if (v[i].x > max_x) max_x = v[i].x;
		if (v[i].x < min_x) min_x = v[i].x;
		if (v[i].y > max_y) max_y = v[i].y;
		if (v[i].y < min_y) min_y = v[i].y;
	}
	if (point.x < min_x || point.x > max_x || point.y < min_y || point.y > max_y) {
		return -1;
	}

	oracle_point_t e = { 2.0 * TUNER_MAX_SIZE, 2.0 * TUNER_MAX_RANKS };
	e = oracle_region_log2(e);

	int crosses = 0;
	for (i = 0; i < n; i++) {
		k = (i + 1) % n;
		if (intersect(point, e, v[i], v[k], eps, 0) == 1) {
			crosses++;
		}
	}
	return (crosses & 1) ? 1 : -1;
}

/* extend_region, :254-289 */
oracle_point_t oracle_region_extend(oracle_point_t a, oracle_point_t b, oracle_point_t z)
{
	oracle_point_t ret;

	a = oracle_region_log2(a);
	b = oracle_region_log2(b);
	z = oracle_region_log2(z);

	if (a.x == b.x) {
		ret.x = a.x, ret.y = z.y;
		return point_pow2(ret);
	}
	if (a.y == b.y) {
		ret.x = z.x, ret.y = a.y;
		return point_pow2(ret);
	}
	double m = (a.y - b.y) / (a.x - b.x);
	double c = b.y - m * b.x;
	double projected_zy = m * z.x + c;

	if (projected_zy < z.y) {
		ret.x = z.x, ret.y = projected_zy;
	} else {
		ret.x = (z.y - c) / m, ret.y = z.y;
	}
	return point_pow2(ret);
}

/* Locate the table rows for (platform, shape, collective); shape selection as
 * in the per-platform init functions (:302,:485; :675,:768,:878; :976,:1182;
 * :1342,:1598): ranks == 8*nodes, ranks == 2*nodes (P5/P5e only), ranks == nodes. */
static int find_set(int platform, uint64_t num_ranks, uint64_t num_nodes, int coll)
{
	int ppn;
	if (num_ranks == 8 * num_nodes) {
		ppn = 8;
	} else if (num_ranks == 2 * num_nodes && platform == ORACLE_PLAT_P5_P5E) {
		ppn = 2;
	} else if (num_ranks == num_nodes) {
		ppn = 1;
	} else {
		return -1;
	}
	for (int s = 0; s < OFI_REGION_NUM_SETS; s++) {
		if (ofi_region_sets[s][0] == platform && ofi_region_sets[s][1] == ppn &&
		    ofi_region_sets[s][2] == coll) {
			return s;
		}
	}
	return -1;
}

/* Build polygon p of set s in log2 space: extension points first (:304-318 and
 * alike), then set_regions' per-vertex transform_log2 (:236-247). */
static int build_poly(int s, int p, oracle_point_t *out)
{
	const int *set = ofi_region_sets[s];
	const int *poly = ofi_region_polys[set[3] + p];
	oracle_point_t ext[8];
	oracle_point_t z = { TUNER_MAX_SIZE, TUNER_MAX_RANKS };

	for (int e = 0; e < set[6]; e++) {
		const double *r = ofi_region_exts[set[5] + e];
		oracle_point_t a = { r[0], r[1] }, b = { r[2], r[3] };
		ext[e] = oracle_region_extend(a, b, z);
	}
	for (int v = 0; v < poly[3]; v++) {
		const int *kind = ofi_region_vert_kind[poly[2] + v];
		const double *xy = ofi_region_vert_xy[poly[2] + v];
		oracle_point_t pt;
		if (kind[0] == 0) {
			pt.x = xy[0];
		} else {
			int e = (kind[0] - 1) / 2;
			pt.x = ((kind[0] - 1) % 2 == 0) ? ext[e].x : ext[e].y;
		}
		if (kind[1] == 0) {
			pt.y = xy[1];
		} else {
			int e = (kind[1] - 1) / 2;
			pt.y = ((kind[1] - 1) % 2 == 0) ? ext[e].x : ext[e].y;
		}
		out[v] = oracle_region_log2(pt);
	}
	return poly[3];
}

int oracle_region_polys(int platform, uint64_t num_ranks, uint64_t num_nodes, int coll,
			int *algos, int *protos, int *nverts, oracle_point_t *verts, int max_polys)
{
	int s = find_set(platform, num_ranks, num_nodes, coll);
	if (s < 0) {
		return 0;
	}
	int np = ofi_region_sets[s][4];
	for (int p = 0; p < np && p < max_polys; p++) {
		const int *poly = ofi_region_polys[ofi_region_sets[s][3] + p];
		algos[p] = poly[0];
		protos[p] = poly[1];
		nverts[p] = build_poly(s, p, &verts[p * MAX_VERTICES]);
	}
	return np;
}

/* log2Down / log2i, include/internal/tuner/nccl_defaults.h:92-104 */
static int log2i(int x)
{
	if (x <= 0) {
		return -1;
	}
	return 31 - __builtin_clz((unsigned int)x);
}

/* calculateChunkSizeTreeLL128, src/tuner/nccl_ofi_regions.cpp:1883-1938;
 * constants from include/internal/tuner/nccl_defaults.h:15-84 */
uint64_t oracle_chunk_tree_ll128(uint64_t message_size, int nChannels, int log2_nnodes)
{
	const int ppn = 8;
	const uint64_t STEPS = 8, LL128_ELEMS_PER_THREAD = 120, LL128_MAX_NTHREADS = 640;
	const uint64_t LINEELEMS = 128 / sizeof(uint64_t), DATAELEMS = LINEELEMS - 1;
	const uint64_t WARP = 32, SHMEM_ELEMS = 8;

	uint64_t buffSize = LL128_ELEMS_PER_THREAD * LL128_MAX_NTHREADS * STEPS * sizeof(uint64_t);
	uint64_t stepSize = buffSize / STEPS;
	uint64_t chunkSize = stepSize;

	chunkSize = (chunkSize / LINEELEMS) * DATAELEMS;
	double nStepsLL128 = 1 + log2_nnodes + 0.1 * ppn;

	while (message_size / (nChannels * chunkSize) < nStepsLL128 * 64 / ppn && chunkSize > 131072) {
		chunkSize /= 2;
	}
	while (message_size / (nChannels * chunkSize) < nStepsLL128 * 16 / ppn && chunkSize > 32768) {
		chunkSize /= 2;
	}

	uint64_t grainSize = (WARP * SHMEM_ELEMS / LINEELEMS * DATAELEMS * sizeof(uint64_t));
	chunkSize = (chunkSize / grainSize) * grainSize;

	uint64_t elementsPerGrain = grainSize / sizeof(float);
	uint64_t chunkGrain = chunkSize / grainSize;
	uint64_t nelem = chunkGrain * elementsPerGrain;

	uint64_t WireWordPerSlice = WARP * SHMEM_ELEMS;
	uint64_t DataEltPerSlice =
		(WireWordPerSlice - WireWordPerSlice / LINEELEMS) * (sizeof(uint64_t) / sizeof(float));

	uint64_t final_chunksize =
		ceil((double)nelem / DataEltPerSlice) * WireWordPerSlice * sizeof(uint64_t);
	return final_chunksize;
}

/* calculateBestNChannelPat, :1943-1953 */
int oracle_best_nchannel_pat(uint64_t message_size, uint64_t num_nodes)
{
	int best = 0;
	if (message_size <= (num_nodes * 65536)) {
		best = 1;
	} else if (message_size <= (num_nodes * 65536 * 2)) {
		best = 2;
	}
	return best;
}

/* calculateBestNChannelTree, :1955-1971 */
int oracle_best_nchannel_tree(uint64_t message_size, int log2_nnodes)
{
	const int channels[] = { 16, 24, 32 };
	int best = 0;
	uint64_t maxChunk = 0;

	for (int i = 0; i < 3; i++) {
		uint64_t payload = oracle_chunk_tree_ll128(message_size, channels[i], log2_nnodes);
		if (payload > maxChunk || (payload == maxChunk && channels[i] > best)) {
			maxChunk = payload;
			best = channels[i];
		}
	}
	return best;
}

/* region_get_coll_info_internal_v3, :2070-2157, on a table with no ignored cell */
void oracle_region_decide(int platform, int coll, uint64_t size, uint64_t num_ranks,
			  uint64_t num_nodes, int *algo_out, int *proto_out, int *nchannels)
{
	oracle_region_decide_masked(platform, coll, size, num_ranks, num_nodes, 0x1fffffu, algo_out,
				    proto_out, nchannels);
}

/* The same with the skip rule spelled out: region i is passed over when bit
 * (algorithm*3 + protocol) of allowed_mask is clear.  v3 clears the bits of cells NCCL
 * marked -1 or that lie beyond numAlgo/numProto (:2109-2114); v2 clears PAT and, without
 * NVLS support, NVLS tree (region_get_coll_info_internal_v2, :2029-2035). */
void oracle_region_decide_masked(int platform, int coll, uint64_t size, uint64_t num_ranks,
				 uint64_t num_nodes, uint32_t allowed_mask, int *algo_out,
				 int *proto_out, int *nchannels)
{
	int in_out = -1;
	int algorithm = -1, protocol = -1;

	*algo_out = -1;
	*proto_out = -1;

	int s = find_set(platform, num_ranks, num_nodes, coll);
	if (s < 0) { /* regions[collType] == NULL, :2084 */
		return;
	}
	if (num_nodes <= 2) { /* :2096 */
		return;
	}
	oracle_point_t p = { (double)size, (double)num_ranks };
	p = oracle_region_log2(p);

	int np = ofi_region_sets[s][4];
	for (int i = 0; i < np && in_out < 0; i++) {
		oracle_point_t verts[MAX_VERTICES];
		const int *poly = ofi_region_polys[ofi_region_sets[s][3] + i];
		algorithm = poly[0];
		protocol = poly[1];
		if (!((allowed_mask >> (algorithm * 3 + protocol)) & 1u)) {
			continue;
		}
		int nv = build_poly(s, i, verts);
		in_out = oracle_region_inside(p, verts, (size_t)nv);
	}
	if (in_out < 0) {
		return;
	}
	*algo_out = algorithm;
	*proto_out = protocol;

	int log2_nnodes = log2i((int)num_nodes); /* :2340 */
	if (platform == ORACLE_PLAT_P6 && size >= 4 * 1024 * 1024 && size <= 32 * 1024 * 1024 &&
	    algorithm == ALGO_TREE && protocol == PROTO_LL128 && num_nodes * 8 == num_ranks) {
		*nchannels = oracle_best_nchannel_tree(size, log2_nnodes);
	}
	if (platform == ORACLE_PLAT_P6 && size <= 32 * 1024 * 1024 && algorithm == ALGO_PAT &&
	    protocol == PROTO_SIMPLE && num_nodes == num_ranks) {
		*nchannels = oracle_best_nchannel_pat(size, num_nodes);
	}
}

/* chunkSizeTuningAllGatherPatSimpleP5en, :2159-2209 */
static uint64_t chunk_ag_pat_simple_p5en(uint64_t nBytes, uint64_t nNodes)
{
	uint64_t sat = nNodes >= 16 ? 524288 : 1048576;
	uint64_t T1 = nNodes >= 16 ? 32 : (nNodes < 8 ? nNodes : 8) + 1;
	uint64_t T2 = nNodes < 16 ? nNodes : 16;
	uint64_t T3 = nNodes < 8 ? nNodes : 8;
	uint64_t tuned = sat;

	while (nBytes / tuned < T1 && tuned > sat / 2) {
		tuned /= 2;
	}
	while (nBytes / tuned < T2 && tuned > 65536) {
		tuned /= 2;
	}
	while (nBytes / tuned < T3 && tuned > 32768) {
		tuned /= 2;
	}
	return tuned;
}

/* chunkSizeTuningTreeLL128P5en, :2211-2274 */
static uint64_t chunk_tree_ll128_p5en(uint64_t nBytes, int log2_nnodes)
{
	uint64_t nsteps = 1 + log2_nnodes;
	uint64_t tuned = 288000;

	if (nBytes / tuned < 2 * nsteps * nsteps) {
		tuned /= 2;
	}
	if (nBytes / tuned < (uint64_t)(1.5 * nsteps)) {
		tuned /= 2;
	}
	while (nBytes / tuned < nsteps + 1 && tuned > 18000) {
		tuned /= 2;
	}
	return tuned;
}

/* region_get_chunk_size_internal, :2276-2306 */
int oracle_region_chunk_size(int platform, int coll, uint64_t size, int algo, int proto,
			     uint64_t num_ranks, uint64_t num_nodes, uint64_t *chunk)
{
	if (num_nodes != num_ranks || platform != ORACLE_PLAT_P5EN) {
		return 0;
	}
	if (coll == FUNC_ALLREDUCE && algo == ALGO_TREE && proto == PROTO_LL128) {
		*chunk = chunk_tree_ll128_p5en(size, log2i((int)num_nodes));
		return 1;
	}
	if (coll == FUNC_ALLGATHER && algo == ALGO_PAT && proto == PROTO_SIMPLE) {
		*chunk = chunk_ag_pat_simple_p5en(size, num_nodes);
		return 1;
	}
	return 0;
}

/* ---- whole-grid loops (the scalar baseline the batched kernels are timed against) ----
 * Layouts as the product's grid entry points: point = ((coll*n_sizes + size)*n_nodes +
 * node)*n_ppn + ppn; cost[point*n_algos*3 + a*3 + proto]; choice[point*2 + {0,1}];
 * region choice[point*3 + {algo, proto, nchannels}] (int32, nchannels -1 when left alone). */
void oracle_model_grid(int platform, int pipe_ops, int num_channels, int net_comp_overhead,
		       const int32_t *colls, uint32_t n_colls, const uint64_t *sizes, uint32_t n_sizes,
		       const uint64_t *nodes, uint32_t n_nodes, const uint32_t *ppn, uint32_t n_ppn,
		       const int32_t *algos, uint32_t n_algos, double *cost, int8_t *choice)
{
	uint64_t point = 0;
	const int modelled = platform == ORACLE_PLAT_P5_P5E || platform == ORACLE_PLAT_P5EN;
	for (uint32_t c = 0; c < n_colls; c++) {
		for (uint32_t s = 0; s < n_sizes; s++) {
			for (uint32_t n = 0; n < n_nodes; n++) {
				for (uint32_t q = 0; q < n_ppn; q++, point++) {
					uint64_t R = nodes[n] * ppn[q];
					if (cost) {
						double *row = cost + point * n_algos * 3;
						for (uint32_t a = 0; a < n_algos; a++) {
							for (int pr = 0; pr < 3; pr++) {
								row[a * 3 + pr] = modelled ? (double)oracle_model_cost(
									platform, colls[c], algos[a], pr, pipe_ops, sizes[s],
									R, nodes[n], num_channels, net_comp_overhead) : -1.0;
							}
						}
					}
					if (choice) {
						int al = -1, pr = -1;
						if (modelled) {
							oracle_model_decide(platform, colls[c], pipe_ops, sizes[s], R,
									    nodes[n], num_channels, net_comp_overhead,
									    &al, &pr);
						}
						choice[point * 2] = (int8_t)al;
						choice[point * 2 + 1] = (int8_t)pr;
					}
				}
			}
		}
	}
}

void oracle_region_grid(int platform, const int32_t *colls, uint32_t n_colls, const uint64_t *sizes,
			uint32_t n_sizes, const uint64_t *nodes, uint32_t n_nodes, const uint32_t *ppn,
			uint32_t n_ppn, int32_t *choice)
{
	uint64_t point = 0;
	for (uint32_t c = 0; c < n_colls; c++) {
		for (uint32_t s = 0; s < n_sizes; s++) {
			for (uint32_t n = 0; n < n_nodes; n++) {
				for (uint32_t q = 0; q < n_ppn; q++, point++) {
					int al, pr, ch = -1;
					oracle_region_decide(platform, colls[c], sizes[s], nodes[n] * ppn[q],
							     nodes[n], &al, &pr, &ch);
					choice[point * 3] = al;
					choice[point * 3 + 1] = pr;
					choice[point * 3 + 2] = ch;
				}
			}
		}
	}
}
