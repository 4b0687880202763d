/*
 * Batched tuner evaluation for gfx950: the cost model and the region lookup over a
 * whole grid of (collective, size, nodes, ranks/node) points in one call.  The
 * arithmetic lives in tuner_device.hpp; this file holds the grid kernels, the plan
 * object and the host-side construction of the log2-space polygon tables
 * (extend_region + set_regions, src/tuner/nccl_ofi_regions.cpp:224-289).
 *
 * Nothing here is matrix-shaped: one thread per decision point, which also evaluates the
 * point's cost cells (staged in LDS, written out as contiguous runs).
 */
#include <algorithm>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "common.hpp"
#include "tuner_device.hpp"
#include "region_tables.inc"

using namespace ofi_amd_tuner;

namespace {

struct grid_dims_t {
	uint32_t n_colls, n_sizes, n_nodes, n_ppn, n_algos;
	const int32_t *colls;
	const uint64_t *sizes;
	const uint64_t *nodes;
	const uint32_t *ppn;
	const int32_t *algos;
	const double *log2_nodes; /* log2((double)nodes[i]) from the host's libm */
	const double *log2_sizes; /* per size index: transform_log2 of the byte count */
	const double *log2_ranks; /* per (node, ppn): transform_log2 of the rank count */
};

/*
 * One thread per decision point; blockIdx.y is the variant.  The thread evaluates the
 * n_algos x 3 cost cells of its point -- contiguous in the output -- and its decision.  Cells
 * are staged in LDS so that the workgroup writes its 256 x cells-per-point doubles as one
 * contiguous run (a lane-per-point store would touch 64 cache lines per instruction).
 */
template <bool COST, bool CHOICE>
__global__ __launch_bounds__(256) void model_grid_kernel(grid_dims_t g,
							 const ofi_amd_tuner_variant_t *__restrict__ variants,
							 uint32_t points_per_variant, double *__restrict__ cost,
							 int8_t *__restrict__ choice)
{
	extern __shared__ double stage[]; /* [256][cells per point] when COST */
	__shared__ int32_t column_of[NUM_ALGOS]; /* the plan's column of an algorithm, -1: none */
	const uint32_t cpp = g.n_algos * NUM_PROTOS;
	const uint32_t first = blockIdx.x * 256u;
	const uint32_t p = first + threadIdx.x;
	const ofi_amd_tuner_variant_t v = variants[blockIdx.y];
	const bool live = p < points_per_variant;
	if (COST && CHOICE) {
		if (threadIdx.x < NUM_ALGOS) {
			int32_t col = -1;
			for (uint32_t ai = g.n_algos; ai-- > 0;) {
				col = g.algos[ai] == (int32_t)threadIdx.x ? (int32_t)ai : col;
			}
			column_of[threadIdx.x] = col;
		}
		__syncthreads();
	}
	if (live) {
		uint32_t r = p;
		const uint32_t pi = r % g.n_ppn; r /= g.n_ppn;
		const uint32_t ni = r % g.n_nodes; r /= g.n_nodes;
		const uint32_t si = r % g.n_sizes; r /= g.n_sizes;
		const uint32_t ci = r;
		const uint64_t nodes = g.nodes[ni];
		const uint64_t per_node = g.ppn[pi];
		const uint64_t ranks = nodes * per_node;
		if (COST) {
			const bool modelled = platform_has_model(v.platform);
			const float size_f = (float)g.sizes[si];
			const int coll = g.colls[ci];
			const double log2_nodes = g.log2_nodes[ni];
			for (uint32_t ai = 0; ai < g.n_algos; ai++) {
				float c[NUM_PROTOS] = { -1.0f, -1.0f, -1.0f };
				if (modelled) {
					/* ranks = nodes * per_node, so ranks / nodes is per_node */
					model_cost_protos(v.platform, coll, g.algos[ai], v.pipe_ops, size_f, ranks, nodes, per_node,
							  log2_nodes, v.num_channels, v.net_comp_overhead, c);
				}
#pragma unroll
				for (uint32_t proto = 0; proto < NUM_PROTOS; proto++) {
					stage[threadIdx.x * cpp + ai * NUM_PROTOS + proto] = (double)c[proto];
				}
			}
		}
		if (CHOICE) {
			int algo, proto;
			if (COST) {
				/* the cells the decision looks at have just been worked out: it reads this thread's
				 * row of the stage instead of evaluating the model again, and goes to the model
				 * only for an algorithm the plan has no column for */
				const double *cells = &stage[threadIdx.x * cpp];
				model_choose_with(
					v.platform, g.colls[ci], g.sizes[si], ranks, nodes, kAllAllowed,
					[&](int a, int pr) -> float {
						const int32_t col = column_of[a];
						if (col >= 0) {
							return (float)cells[col * NUM_PROTOS + pr]; /* exact: it was a float */
						}
						return model_cost(v.platform, g.colls[ci], a, pr, v.pipe_ops, g.sizes[si], ranks,
								  nodes, g.log2_nodes[ni], v.num_channels, v.net_comp_overhead);
					},
					algo, proto);
			} else {
				model_choose(v.platform, g.colls[ci], g.sizes[si], ranks, nodes, g.log2_nodes[ni], v.pipe_ops,
					     v.num_channels, v.net_comp_overhead, kAllAllowed, algo, proto);
			}
			const uint64_t at = ((uint64_t)blockIdx.y * points_per_variant + p) * 2u;
			if ((reinterpret_cast<uintptr_t>(choice) & 1u) == 0) {
				*reinterpret_cast<uint16_t *>(choice + at) =
					(uint16_t)((uint8_t)(int8_t)algo | ((uint32_t)(uint8_t)(int8_t)proto << 8));
			} else {
				choice[at + 0] = (int8_t)algo;
				choice[at + 1] = (int8_t)proto;
			}
		}
	}
	if (COST) {
		__syncthreads();
		const uint32_t valid = min(256u, points_per_variant - first);
		double *out = cost + ((uint64_t)blockIdx.y * points_per_variant + first) * cpp;
		const uint32_t cells = valid * cpp;
		if ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
			/* two cells per lane and store: 1 KiB per wavefront instruction */
			typedef double double2_t __attribute__((ext_vector_type(2)));
			const double2_t *from = reinterpret_cast<const double2_t *>(stage);
			double2_t *to = reinterpret_cast<double2_t *>(out);
			for (uint32_t k = threadIdx.x; k < cells / 2; k += 256u) {
				__builtin_nontemporal_store(from[k], &to[k]);
			}
			if ((cells & 1u) && threadIdx.x == 0) {
				out[cells - 1] = stage[cells - 1];
			}
		} else {
			for (uint32_t k = threadIdx.x; k < cells; k += 256u) {
				__builtin_nontemporal_store(stage[k], &out[k]);
			}
		}
	}
}

constexpr int kMaxSetPolys = 8;  /* polygons of one (platform, shape, collective) set */
constexpr int kMaxSetVerts = 64; /* their vertices together */
constexpr uint32_t kRegionBlock = 64; /* threads per workgroup of the region kernel: one wavefront */
constexpr uint32_t kXcds = 8;         /* workgroup w of a launch runs on XCD w mod 8, each with its own L2 */
static_assert(kRegionBlock >= (uint32_t)kMaxSetVerts && kRegionBlock >= (uint32_t)kMaxSetPolys * 4,
	      "one thread per staged vertex and per staged polygon word");

/*
 * One thread per point.  A workgroup (one wavefront) works on 64 points of one (collective,
 * ranks per node) pair -- `blocks_per_run` chunks make up the pair's n_sizes x n_nodes points,
 * node count fastest -- because the polygon set depends on that pair alone: the set (at most 8 polygons, 64 vertices, with their bounds) is copied into LDS
 * once and every lane then walks the same polygons out of LDS instead of chasing them through
 * global memory, and workgroups of pairs without regions leave after one table lookup.
 *
 * In the output the ranks-per-node index runs fastest, so a wavefront's 64 records lie 4 x
 * n_ppn bytes apart and the records between them belong to the same chunk's other
 * ranks-per-node values, i.e. to other workgroups.  Those workgroups are given numbers that
 * are equal mod 8: they run on the same XCD, their partial writes to a cache line meet in that
 * XCD's L2 and leave it as one line (measured: 4.7 MB written for 4.7 MB of records; with the
 * workgroups of a chunk on different XCDs every L2 wrote its quarter of each line, 18.9 MB).
 * Giving a thread all ranks-per-node values of its point, or a workgroup four wavefronts that
 * share an LDS staging buffer, writes the same 4.7 MB but makes the units of work four times
 * coarser, and the launch, which lasts as long as its most loaded SIMD, 15-18 % longer than
 * with single-wavefront units.
 */
__global__ __launch_bounds__(kRegionBlock) void region_choice_kernel(grid_dims_t g, region_tables_t t,
							    const int32_t *__restrict__ platforms,
							    uint32_t points_per_platform, uint32_t blocks_per_run,
							    const uint2 *__restrict__ order, int8_t *__restrict__ choice)
{
	__shared__ int32_t s_poly[kMaxSetPolys * 4];
	__shared__ double s_bounds[kMaxSetPolys * 4];
	__shared__ pt_t s_verts[kMaxSetVerts];

	/* blockIdx.x = k * 8 + x (a one-dimensional grid, so x is the XCD).  order[k] names a
	 * (platform entry, group, pi): chunk 8 * group + x' of the collectives' chunks,
	 * ranks-per-node index pi -- whatever the order, the workgroups of one chunk and platform
	 * entry share x.  The host lists the triples by falling cost (polygons of the pair's set):
	 * the long workgroups start first and the short ones fill the end of the launch, and
	 * workgroups of equal cost are neighbours in launch order, which the dispatcher deals to
	 * the CUs of an XCD in turn.  (In (entry, group, pi) order, or scattered by a fixed stride,
	 * the pairs with many regions recur at periods that keep meeting the same CUs: 74-78 us
	 * against 54 us.) */
	const uint32_t x = blockIdx.x % kXcds;
	const uint2 item = order[blockIdx.x / kXcds];
	const uint32_t entry = item.x;
	const uint32_t pi = item.y % g.n_ppn;
	const uint32_t group = item.y / g.n_ppn;
	/* which of a group's eight chunks an XCD takes rotates with the platform entry: the chunks
	 * differ in cost (collective, size range), and an XCD that kept the same ones for every
	 * entry would keep the same share of the long ones */
	const uint32_t chunk = group * kXcds + (x + entry) % kXcds;
	if (chunk >= blocks_per_run * g.n_colls) {
		return; /* padding of the last group */
	}
	const uint32_t ci = chunk / blocks_per_run;
	const uint32_t in_run = (chunk - ci * blocks_per_run) * kRegionBlock + threadIdx.x;
	const int platform = platforms[entry];
	const int coll = g.colls[ci];
	const uint32_t ppn = g.ppn[pi];

	/* ranks = nodes * ppn with nodes >= 1: the shape is a function of ppn */
	int first, count;
	region_set(t, platform, coll, ppn, 1, first, count);
	if (count > 0) {
		const int v0 = t.poly[first * 4 + 2];
		const int v_end = t.poly[(first + count - 1) * 4 + 2] + t.poly[(first + count - 1) * 4 + 3];
		if ((int)threadIdx.x < count * 4) {
			const int32_t w = t.poly[first * 4 + threadIdx.x];
			s_poly[threadIdx.x] = (threadIdx.x & 3u) == 2u ? w - v0 : w; /* vertex index within the set */
			s_bounds[threadIdx.x] = t.bbox[first * 4 + threadIdx.x];
		}
		if ((int)threadIdx.x < v_end - v0) {
			s_verts[threadIdx.x] = t.verts[v0 + threadIdx.x];
		}
		__syncthreads();
	}
	if (in_run >= g.n_sizes * g.n_nodes) {
		return;
	}
	const uint32_t ni = in_run % g.n_nodes;
	const uint32_t si = in_run / g.n_nodes;
	const uint32_t p = ((ci * g.n_sizes + si) * g.n_nodes + ni) * g.n_ppn + pi; /* output order */

	const uint64_t nodes = g.nodes[ni];
	int algorithm = -1, protocol = -1, nchannels = -1;
	if (count > 0 && nodes > 2) {
		int a, pr;
		const pt_t at = { g.log2_sizes[si], g.log2_ranks[ni * g.n_ppn + pi] };
		if (region_pick(s_poly, s_bounds, s_verts, count, at, kAllAllowed, t.far_point, a, pr) >= 0) {
			algorithm = a;
			protocol = pr;
			nchannels = region_channels(platform, g.sizes[si], nodes * ppn, nodes, a, pr);
		}
	}
	const uint64_t idx = (uint64_t)entry * points_per_platform + p;
	/* {int8 algorithm, int8 protocol, int16 nchannels} as one 4-byte store */
	reinterpret_cast<uint32_t *>(choice)[idx] = ((uint32_t)(uint8_t)(int8_t)algorithm) |
						     ((uint32_t)(uint8_t)(int8_t)protocol << 8) |
						     ((uint32_t)(uint16_t)(int16_t)nchannels << 16);
}

/* ---- host side: building the log2-space polygon tables ---- */

constexpr double kTunerMaxRanks = 1024.0 * 1024;               /* nccl_ofi_tuner_region.h:69 */
constexpr double kTunerMaxSize = 100.0 * 1024 * 1024 * 1024;   /* :74 */

/* transform_log2, include/tuner/nccl_ofi_tuner_region.h:87-109 */
pt_t to_log2(pt_t p)
{
	return pt_t{ log2_coord(p.x), log2_coord(p.y) };
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

int build_region_tables(region_tables_t *t)
{
	std::vector<int32_t> poly;
	std::vector<pt_t> verts;
	std::vector<double> bounds;
	for (int p = 0; p < kNumPlatforms; p++) {
		for (int s = 0; s < kNumShapes; s++) {
			for (int c = 0; c < NUM_FUNCS; c++) {
				t->set_first[p][s][c] = 0;
				t->set_count[p][s][c] = 0;
			}
		}
	}
	const pt_t z = { kTunerMaxSize, kTunerMaxRanks };
	for (int s = 0; s < OFI_REGION_NUM_SETS; s++) {
		const int *set = ofi_region_sets[s];
		const int shape = set[1] == 8 ? 0 : (set[1] == 2 ? 1 : 2);
		pt_t ext[8];
		if (set[6] > 8) {
			return -EINVAL;
		}
		for (int e = 0; e < set[6]; e++) {
			const double *r = ofi_region_exts[set[5] + e];
			ext[e] = extend(pt_t{ r[0], r[1] }, pt_t{ r[2], r[3] }, z);
		}
		t->set_first[set[0]][shape][set[2]] = (int32_t)(poly.size() / 4);
		t->set_count[set[0]][shape][set[2]] = set[4];
		const size_t set_first_vertex = verts.size();
		if (set[4] > kMaxSetPolys) {
			return -EINVAL;
		}
		for (int q = 0; q < set[4]; q++) {
			const int *pd = ofi_region_polys[set[3] + q];
			if (pd[3] < 2 || pd[3] > kMaxVertices) {
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
				verts.push_back(to_log2(pt)); /* set_regions, :236-247 */
			}
			double b[4];
			region_bounds(&verts[verts.size() - pd[3]], pd[3], b);
			bounds.insert(bounds.end(), b, b + 4);
		}
		if (verts.size() - set_first_vertex > (size_t)kMaxSetVerts) {
			return -EINVAL; /* the grid kernel keeps one set in LDS */
		}
	}
	t->far_point = to_log2(pt_t{ 2.0 * kTunerMaxSize, 2.0 * kTunerMaxRanks });
	int32_t *d_poly = nullptr;
	pt_t *d_verts = nullptr;
	double *d_bounds = nullptr;
	int rc = upload(poly, &d_poly);
	if (rc == 0) {
		rc = upload(verts, &d_verts);
	}
	if (rc == 0) {
		rc = upload(bounds, &d_bounds);
	}
	if (rc != 0) {
		(void)hipFree(d_poly);
		(void)hipFree(d_verts);
		return rc;
	}
	t->poly = d_poly;
	t->verts = d_verts;
	t->bbox = d_bounds;
	return 0;
}

} // namespace

namespace ofi_amd_tuner {

double log2_coord(double v)
{
	if (v == 0) {
		v = 1e-6; /* "for 0, set to a small positive number for log2()" */
	}
	return std::log2(v);
}

/* Built once per process (about 13 KiB of device memory, never freed).  A failed build is
 * not remembered: the next caller tries again. */
int device_region_tables(region_tables_t *out)
{
	/* one copy of the tables per GPU, uploaded to whichever is current on first use there */
	constexpr int kMaxDevices = 64;
	static std::mutex lock;
	static region_tables_t tables[kMaxDevices];
	static bool built[kMaxDevices];
	int dev = -1;
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
		(void)hipGetLastError();
		return -ENODEV;
	}
	std::lock_guard<std::mutex> g(lock);
	if (!built[dev]) {
		const int status = build_region_tables(&tables[dev]);
		if (status != 0) {
			return status;
		}
		built[dev] = true;
	}
	*out = tables[dev];
	return 0;
}

} // namespace ofi_amd_tuner

struct ofi_amd_tuner_plan {
	grid_dims_t g;
	region_tables_t t;
	uint64_t points;
	uint64_t cells;
	/* owned device allocations */
	int32_t *d_colls, *d_algos;
	uint64_t *d_sizes, *d_nodes;
	uint32_t *d_ppn;
	double *d_log2_nodes, *d_log2_sizes, *d_log2_ranks;
	/* per-call variant / platform staging (device) */
	ofi_amd_tuner_variant_t *d_variants;
	int32_t *d_platforms;
	uint32_t variants_cap, platforms_cap;
	/* what d_variants currently holds, so that an unchanged list is not uploaded again */
	std::vector<ofi_amd_tuner_variant_t> h_variants;
	std::vector<int32_t> h_platforms;
	/* region launch order for the current platform list (see region_choice_kernel) */
	std::vector<int32_t> h_colls;
	std::vector<uint32_t> h_ppn;
	uint2 *d_order;
	uint64_t order_cap;
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
	(void)hipFree(plan->d_sizes);
	(void)hipFree(plan->d_nodes);
	(void)hipFree(plan->d_ppn);
	(void)hipFree(plan->d_log2_nodes);
	(void)hipFree(plan->d_log2_sizes);
	(void)hipFree(plan->d_log2_ranks);
	(void)hipFree(plan->d_variants);
	(void)hipFree(plan->d_platforms);
	(void)hipFree(plan->d_order);
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
	/* value-initialised: every pointer and capacity starts at zero */
	if (!plan) {
		return -ENOMEM;
	}
	rc = device_region_tables(&plan->t);
	if (rc != 0) {
		delete plan;
		return rc;
	}

	/* query coordinates, through the host's libm */
	std::vector<double> log2_nodes(n_nodes), log2_sizes(n_sizes), log2_ranks((size_t)n_nodes * n_ppn);
	for (uint32_t i = 0; i < n_nodes; i++) {
		log2_nodes[i] = std::log2((double)nodes[i]);
		for (uint32_t j = 0; j < n_ppn; j++) {
			log2_ranks[(size_t)i * n_ppn + j] = log2_coord((double)(nodes[i] * ppn[j]));
		}
	}
	for (uint32_t i = 0; i < n_sizes; i++) {
		log2_sizes[i] = log2_coord((double)sizes[i]);
	}

	rc = upload(std::vector<int32_t>(colls, colls + n_colls), &plan->d_colls);
	if (rc == 0) rc = upload(std::vector<int32_t>(algos, algos + n_algos), &plan->d_algos);
	if (rc == 0) rc = upload(std::vector<uint64_t>(sizes, sizes + n_sizes), &plan->d_sizes);
	if (rc == 0) rc = upload(std::vector<uint64_t>(nodes, nodes + n_nodes), &plan->d_nodes);
	if (rc == 0) rc = upload(std::vector<uint32_t>(ppn, ppn + n_ppn), &plan->d_ppn);
	if (rc == 0) rc = upload(log2_nodes, &plan->d_log2_nodes);
	if (rc == 0) rc = upload(log2_sizes, &plan->d_log2_sizes);
	if (rc == 0) rc = upload(log2_ranks, &plan->d_log2_ranks);
	if (rc != 0) {
		ofi_amd_tuner_plan_destroy(plan);
		return rc;
	}

	try {
		plan->h_colls.assign(colls, colls + n_colls);
		plan->h_ppn.assign(ppn, ppn + n_ppn);
	} catch (...) {
		ofi_amd_tuner_plan_destroy(plan);
		return -ENOMEM;
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
	g.log2_sizes = plan->d_log2_sizes;
	g.log2_ranks = plan->d_log2_ranks;
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
		plan->h_variants.clear();
		OFI_AMD_HIP_TRY(hipMalloc((void **)&plan->d_variants, sizeof(*variants) * n_variants));
		plan->variants_cap = n_variants;
	}
	/* the variants travel to the device only when they differ from the last call's */
	try {
		if (plan->h_variants.size() != n_variants ||
		    std::memcmp(plan->h_variants.data(), variants, sizeof(*variants) * n_variants) != 0) {
			plan->h_variants.assign(variants, variants + n_variants);
			OFI_AMD_HIP_TRY(hipMemcpyAsync(plan->d_variants, plan->h_variants.data(),
						       sizeof(*variants) * n_variants, hipMemcpyHostToDevice, s));
			/* the source is pageable host memory owned by the plan: wait until it has been read */
			OFI_AMD_HIP_TRY(hipStreamSynchronize(s));
		}
	} catch (...) {
		return -ENOMEM;
	}
	if (plan->points > (1ull << 31) || plan->cells * n_variants > (1ull << 38) || n_variants > 65535) {
		return -EINVAL;
	}
	const uint32_t points = (uint32_t)plan->points;
	const dim3 grid((points + 255u) / 256u, n_variants);
	const size_t lds = (size_t)256 * plan->g.n_algos * NUM_PROTOS * sizeof(double);
	if (d_cost && d_choice) {
		hipLaunchKernelGGL((model_grid_kernel<true, true>), grid, dim3(256), lds, s, plan->g,
				   plan->d_variants, points, d_cost, d_choice);
	} else if (d_cost) {
		hipLaunchKernelGGL((model_grid_kernel<true, false>), grid, dim3(256), lds, s, plan->g,
				   plan->d_variants, points, d_cost, d_choice);
	} else if (d_choice) {
		hipLaunchKernelGGL((model_grid_kernel<false, true>), grid, dim3(256), 0, s, plan->g,
				   plan->d_variants, points, d_cost, d_choice);
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
	if (!plan || !platforms || n_platforms == 0 || !d_choice || (reinterpret_cast<uintptr_t>(d_choice) & 3u) != 0) {
		return -EINVAL;
	}
	for (uint32_t i = 0; i < n_platforms; i++) {
		if (platforms[i] < 0 || platforms[i] >= kNumPlatforms) {
			return -EINVAL;
		}
	}
	if (plan->points > (1ull << 31) || n_platforms > 65535) {
		return -EINVAL;
	}
	const uint32_t points = (uint32_t)plan->points;
	const uint64_t run_len = (uint64_t)plan->g.n_sizes * plan->g.n_nodes;
	const uint64_t blocks_per_run = (run_len + kRegionBlock - 1) / kRegionBlock;
	const uint64_t n_chunks = blocks_per_run * plan->g.n_colls;
	const uint64_t n_groups = (n_chunks + kXcds - 1) / kXcds;
	const uint64_t per_entry = n_groups * plan->g.n_ppn;
	const uint64_t per_xcd = per_entry * n_platforms;
	const uint64_t blocks = per_xcd * kXcds;
	if (blocks == 0 || blocks > 0x7fffffffull) {
		return -EINVAL;
	}

	hipStream_t s = as_stream(stream);
	if (n_platforms > plan->platforms_cap || per_xcd > plan->order_cap) {
		OFI_AMD_HIP_TRY(hipStreamSynchronize(s));
		(void)hipFree(plan->d_platforms);
		(void)hipFree(plan->d_order);
		plan->d_platforms = nullptr;
		plan->d_order = nullptr;
		plan->platforms_cap = 0;
		plan->order_cap = 0;
		plan->h_platforms.clear();
		OFI_AMD_HIP_TRY(hipMalloc((void **)&plan->d_platforms, sizeof(int32_t) * n_platforms));
		plan->platforms_cap = n_platforms;
		OFI_AMD_HIP_TRY(hipMalloc((void **)&plan->d_order, sizeof(uint2) * per_xcd));
		plan->order_cap = per_xcd;
	}
	try {
		if (plan->h_platforms.size() != n_platforms ||
		    std::memcmp(plan->h_platforms.data(), platforms, sizeof(int32_t) * n_platforms) != 0) {
			plan->h_platforms.clear(); /* stays empty if an upload fails: the next call uploads again */
			/* launch order: (entry, group, pi) by falling number of polygons in the pair's set; a
			 * group that straddles two collectives counts as the costlier one */
			struct item_t {
				int32_t cost;
				uint2 v;
			};
			std::vector<item_t> items;
			items.reserve(per_xcd);
			for (uint32_t pi = 0; pi < plan->g.n_ppn; pi++) {
				for (uint64_t group = 0; group < n_groups; group++) {
					const uint64_t last = std::min<uint64_t>(group * kXcds + kXcds - 1, n_chunks - 1);
					const int32_t c0 = plan->h_colls[group * kXcds / blocks_per_run];
					const int32_t c1 = plan->h_colls[last / blocks_per_run];
					for (uint32_t e = 0; e < n_platforms; e++) {
						int first, count0, count1;
						region_set(plan->t, platforms[e], c0, plan->h_ppn[pi], 1, first, count0);
						region_set(plan->t, platforms[e], c1, plan->h_ppn[pi], 1, first, count1);
						items.push_back({ std::max(count0, count1),
								  make_uint2(e, (uint32_t)(group * plan->g.n_ppn + pi)) });
					}
				}
			}
			std::stable_sort(items.begin(), items.end(),
					 [](const item_t &a, const item_t &b) { return a.cost > b.cost; });
			std::vector<uint2> order(items.size());
			for (size_t i = 0; i < items.size(); i++) {
				order[i] = items[i].v;
			}
			OFI_AMD_HIP_TRY(hipMemcpyAsync(plan->d_platforms, platforms, sizeof(int32_t) * n_platforms,
						       hipMemcpyHostToDevice, s));
			OFI_AMD_HIP_TRY(hipMemcpyAsync(plan->d_order, order.data(), sizeof(uint2) * order.size(),
						       hipMemcpyHostToDevice, s));
			OFI_AMD_HIP_TRY(hipStreamSynchronize(s));
			plan->h_platforms.assign(platforms, platforms + n_platforms);
		}
	} catch (...) {
		plan->h_platforms.clear();
		return -ENOMEM;
	}
	hipLaunchKernelGGL(region_choice_kernel, dim3((uint32_t)blocks), dim3(kRegionBlock), 0, s, plan->g, plan->t,
			   plan->d_platforms, points, (uint32_t)blocks_per_run, plan->d_order, d_choice);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

} /* extern "C" */
