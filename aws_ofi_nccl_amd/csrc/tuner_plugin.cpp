/*
 * NCCL / RCCL tuner plugin symbols on top of the GPU tuner: ncclTunerPlugin_v2, _v3 and
 * _v6 with the behaviour of src/tuner/nccl_ofi_tuner.cpp:29-279 in the reference.
 *
 * NCCL calls getCollInfo once per collective launch, at enqueue time -- possibly inside a
 * stream capture -- and a training job repeats the same few (collective, size) pairs.  So
 * init does everything that allocates (the query stream, its pinned staging, the region
 * tables in device memory) and evaluates, in one batched launch, the power-of-two size
 * ladder of every collective for the communicator's shape; after that a question is served
 * from the per-communicator table, and only a size off the ladder costs a GPU round trip
 * (a launch on a private stream and a wait, no allocation), once.  There is no host
 * evaluation path: without a usable GPU init fails, and a query that fails later hands the
 * decision back to NCCL's own tuner.
 *
 * Platform selection follows include/tuner/nccl_ofi_tuner_process_config.h:17-116: the
 * EC2 product name (OFI_NCCL_FORCE_PRODUCT_NAME, else the DMI product_name file,
 * src/nccl_ofi_system.cpp:110-160) picks one of four tables; OFI_NCCL_TUNER_TYPE
 * (Internal | Region | Model, case-insensitive) and a set OFI_NCCL_FORCE_NUM_RAILS can
 * hand the decision back to NCCL.  The hwloc / libfabric topology probe the reference
 * runs before that is not reproduced.
 */
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include <strings.h>

#include "nccl_tuner_abi.h"
#include "ofi_amd_hotpath.h"

namespace {

constexpr uint32_t kAllAllowed = (1u << (NCCL_NUM_ALGORITHMS * NCCL_NUM_PROTOCOLS)) - 1;
constexpr int kAlgoNvlsTree = 5, kAlgoPat = 6;

ncclDebugLogger_t g_log = nullptr;
std::mutex g_ctx_lock; /* nccl_ofi_tuner_ctx_lock */

#define TUNER_INFO(...)                                                                         \
	do {                                                                                    \
		if (g_log) g_log(NCCL_LOG_INFO, NCCL_INIT | NCCL_TUNING, __FILE__, __LINE__, __VA_ARGS__); \
	} while (0)
#define TUNER_WARN(...)                                                                         \
	do {                                                                                    \
		if (g_log) g_log(NCCL_LOG_WARN, ~0ul, __FILE__, __LINE__, __VA_ARGS__);         \
	} while (0)

struct key_t {
	uint64_t nbytes;
	uint32_t mask;
	int32_t kind, coll, pipe_ops, algo, proto;
	bool operator==(const key_t &o) const
	{
		return nbytes == o.nbytes && mask == o.mask && kind == o.kind && coll == o.coll &&
		       pipe_ops == o.pipe_ops && algo == o.algo && proto == o.proto;
	}
};
struct key_hash {
	size_t operator()(const key_t &k) const
	{
		uint64_t h = k.nbytes * 0x9E3779B97F4A7C15ull;
		h ^= ((uint64_t)k.mask << 32 | (uint32_t)k.coll) * 0xBF58476D1CE4E5B9ull;
		h ^= ((uint64_t)(uint32_t)k.pipe_ops << 32 | (uint32_t)(k.kind * 64 + k.algo * 4 + k.proto)) *
		     0x94D049BB133111EBull;
		return (size_t)(h ^ (h >> 29));
	}
};

constexpr uint32_t kCtxMagic = 0x544e5543u;

struct tuner_ctx {
	uint32_t magic = kCtxMagic;
	int platform;
	int model; /* 0: region tuner, 1: model tuner */
	uint64_t ranks, nodes;
	int num_channels, net_comp_overhead;
	std::mutex lock;
	std::unordered_map<key_t, ofi_amd_tuner_answer_t, key_hash> memo;
	ofi_amd_tuner_ctx_stats_t stats = {};
};

constexpr int kMaxPreloadPipeOps = 4; /* numPipeOps values evaluated ahead for the model tuner */
constexpr uint32_t kPreloadCapacity = 1024;

void fill_query(const tuner_ctx *ctx, const key_t &key, ofi_amd_tuner_query_t *q)
{
	std::memset(q, 0, sizeof(*q));
	q->platform = ctx->platform;
	q->kind = key.kind;
	q->coll = key.coll;
	q->pipe_ops = key.pipe_ops;
	q->num_channels = ctx->num_channels;
	q->net_comp_overhead = ctx->net_comp_overhead;
	q->algo = key.algo;
	q->proto = key.proto;
	q->allowed_mask = key.mask;
	q->nbytes = key.nbytes;
	q->num_ranks = ctx->ranks;
	q->num_nodes = ctx->nodes;
}

/* The questions a job typically asks first: every collective at the powers of two from 1 B to
 * 64 GiB with nothing ruled out, and the chunk sizes of the two tuned (collective, algorithm,
 * protocol) combinations, in one launch. */
int preload(tuner_ctx *ctx)
{
	std::vector<key_t> keys;
	try {
		for (int coll = 0; coll < NCCL_NUM_FUNCTIONS; coll++) {
			for (int e = 0; e <= 36; e++) {
				const uint64_t nbytes = 1ull << e;
				if (ctx->model) {
					for (int pipe = 1; pipe <= kMaxPreloadPipeOps; pipe++) {
						keys.push_back(key_t{ nbytes, kAllAllowed, 1, coll, pipe, 0, 0 });
					}
				} else {
					keys.push_back(key_t{ nbytes, kAllAllowed, 0, coll, 0, 0, 0 });
				}
			}
		}
		if (!ctx->model) {
			for (int e = 0; e <= 36; e++) {
				keys.push_back(key_t{ 1ull << e, kAllAllowed, 2, 4 /* AllReduce */, 0, 0 /* Tree */, 1 /* LL128 */ });
				keys.push_back(key_t{ 1ull << e, kAllAllowed, 2, 2 /* AllGather */, 0, kAlgoPat, 2 /* Simple */ });
			}
		}
		std::vector<ofi_amd_tuner_query_t> qs(keys.size());
		std::vector<ofi_amd_tuner_answer_t> as(keys.size());
		for (size_t i = 0; i < keys.size(); i++) {
			fill_query(ctx, keys[i], &qs[i]);
		}
		const int rc = ofi_amd_tuner_query(qs.data(), (uint32_t)qs.size(), as.data());
		if (rc != 0) {
			return rc;
		}
		for (size_t i = 0; i < keys.size(); i++) {
			ctx->memo.emplace(keys[i], as[i]);
		}
		ctx->stats.preloaded = keys.size();
	} catch (...) {
		return -ENOMEM;
	}
	return 0;
}

/* nccl_net_ofi_get_product_name, src/nccl_ofi_system.cpp:110-160 */
std::string product_name()
{
	if (const char *forced = getenv("OFI_NCCL_FORCE_PRODUCT_NAME")) {
		return forced;
	}
	std::string name;
	if (FILE *f = fopen("/sys/devices/virtual/dmi/id/product_name", "r")) {
		char buf[64] = { 0 };
		if (fgets(buf, sizeof(buf), f)) {
			name = buf;
			while (!name.empty() && (name.back() == '\n' || name.back() == ' ')) {
				name.pop_back();
			}
		}
		fclose(f);
	}
	return name;
}

int platform_of(const std::string &name)
{
	if (name == "p5.48xlarge" || name == "p5e.48xlarge") return OFI_AMD_PLATFORM_P5_P5E;
	if (name == "p5en.48xlarge") return OFI_AMD_PLATFORM_P5EN;
	if (name == "p6-b200.48xlarge") return OFI_AMD_PLATFORM_P6;
	if (name == "p6-b300.48xlarge") return OFI_AMD_PLATFORM_P6_B300;
	return -1;
}

int env_int(const char *name, int fallback)
{
	const char *v = getenv(name);
	if (!v || !*v) {
		return fallback;
	}
	char *end = nullptr;
	long x = strtol(v, &end, 10);
	return (end && *end == '\0') ? (int)x : fallback;
}

ncclResult_t tuner_destroy(void *context)
{
	std::lock_guard<std::mutex> g(g_ctx_lock);
	delete static_cast<tuner_ctx *>(context);
	return ncclSuccess;
}

/* nccl_ofi_tuner_init, src/tuner/nccl_ofi_tuner.cpp:47-136 */
ncclResult_t tuner_init(size_t nRanks, size_t nNodes, ncclDebugLogger_t logFunction, void **context)
{
	*context = nullptr;
	if (!g_log) {
		g_log = logFunction;
	}
	std::lock_guard<std::mutex> g(g_ctx_lock);

	const std::string name = product_name();
	const char *type = getenv("OFI_NCCL_TUNER_TYPE");
	const bool internal = type && strcasecmp(type, "INTERNAL") == 0;
	const bool force_model = type && strcasecmp(type, "MODEL") == 0;
	if (name.empty()) {
		TUNER_INFO("NCCL_OFI_TUNER is not available because platform type is unavailable.");
		return ncclSuccess;
	}
	if (internal) {
		TUNER_INFO("NCCL_OFI_TUNER_TYPE is Internal, Fall back to NCCL's tuner for platform : %s",
			   name.c_str());
		return ncclSuccess;
	}
	if (getenv("OFI_NCCL_FORCE_NUM_RAILS")) {
		TUNER_INFO("Falling back to NCCL's tuner due to OFI_NCCL_FORCE_NUM_RAILS being set.");
		return ncclSuccess;
	}
	const int platform = platform_of(name);
	if (platform < 0) { /* neither region nor model tables for it */
		TUNER_INFO("NCCL_OFI_TUNER is not available for platform : %s, Fall back to NCCL's tuner",
			   name.c_str());
		return ncclSuccess;
	}
	const bool model_support = platform == OFI_AMD_PLATFORM_P5_P5E || platform == OFI_AMD_PLATFORM_P5EN;

	int rc = ofi_amd_gpu_init();
	if (rc != 0) {
		TUNER_WARN("GPU tuner unavailable (ofi_amd_gpu_init: %d)", rc);
		return ncclSystemError;
	}
	/* everything the later queries need is created here, not inside a getCollInfo call */
	rc = ofi_amd_tuner_query_prepare(kPreloadCapacity);
	if (rc != 0) {
		TUNER_WARN("GPU tuner unavailable (ofi_amd_tuner_query_prepare: %d)", rc);
		return ncclSystemError;
	}
	auto *ctx = new (std::nothrow) tuner_ctx();
	if (!ctx) {
		TUNER_WARN("Context allocation failed.");
		return ncclInternalError;
	}
	ctx->platform = platform;
	ctx->model = (model_support && force_model) ? 1 : 0; /* Region wins when both apply (:102-107) */
	ctx->ranks = nRanks;
	ctx->nodes = nNodes;
	ctx->num_channels = env_int("OFI_NCCL_TUNER_NUM_CHANNELS", 8);
	ctx->net_comp_overhead = env_int("OFI_NCCL_TUNER_NET_COMP_OVERHEAD", 3);
	TUNER_INFO("%s base Tuner is chosen for platform: %s", ctx->model ? "Model" : "Region", name.c_str());
	TUNER_INFO("Tuner init: comm with %ld ranks and %ld nodes.", (long)nRanks, (long)nNodes);
	if (nRanks > 0 && nNodes > 0) {
		rc = preload(ctx);
		if (rc != 0) {
			TUNER_WARN("GPU tuner pre-evaluation failed: %d", rc);
			delete ctx;
			return ncclSystemError;
		}
	}
	*context = ctx;
	return ncclSuccess;
}

ncclResult_t tuner_init_v2(size_t nRanks, size_t nNodes, ncclDebugLogger_t logFunction, void **context)
{
	if (getenv("NCCL_ALGO") || getenv("NCCL_PROTO")) { /* :143-155 */
		if (!g_log) {
			g_log = logFunction;
		}
		TUNER_INFO("The tuner plugin can not be loaded when explicitly choosing an algorithm or "
			   "protocol with NCCL_ALGO/NCCL_PROTO. Defaulting to internal tuner.");
		*context = nullptr;
		return ncclSuccess;
	}
	return tuner_init(nRanks, nNodes, logFunction, context);
}

ncclResult_t tuner_init_v6(void **ctx, uint64_t, size_t nRanks, size_t nNodes, ncclDebugLogger_t logFunction,
			   ncclNvlDomainInfo_v6_t *, ncclTunerConstants_v6_t *)
{
	return tuner_init(nRanks, nNodes, logFunction, ctx);
}

/* One question, answered by the GPU the first time and from the table afterwards. */
int ask(tuner_ctx *ctx, int kind, int coll, uint64_t nbytes, int pipe_ops, uint32_t mask, int algo,
	int proto, ofi_amd_tuner_answer_t *out)
{
	const key_t key = { nbytes, mask, kind, coll, pipe_ops, algo, proto };
	std::lock_guard<std::mutex> g(ctx->lock);
	auto it = ctx->memo.find(key);
	if (it != ctx->memo.end()) {
		*out = it->second;
		ctx->stats.hits++;
		return 0;
	}
	if (kind != 2 && mask != kAllAllowed) {
		/* The answer with nothing ruled out also holds under a narrower mask that still
		 * allows the chosen cell: the region tuner takes the first region in table order
		 * that holds the point and is allowed (src/tuner/nccl_ofi_regions.cpp:2106-2128),
		 * so if the first region that holds the point is allowed it stays the answer, and
		 * if no region holds the point none does under any mask; the model tuner's minimum
		 * over all cells stays the minimum when a cell other than it is taken away. */
		key_t open = key;
		open.mask = kAllAllowed;
		it = ctx->memo.find(open);
		if (it != ctx->memo.end()) {
			const ofi_amd_tuner_answer_t &a = it->second;
			if (a.algo < 0 || ((mask >> (a.algo * NCCL_NUM_PROTOCOLS + a.proto)) & 1u)) {
				*out = a;
				ctx->stats.hits++;
				return 0;
			}
		}
	}
	ctx->stats.misses++;
	ofi_amd_tuner_query_t q;
	fill_query(ctx, key, &q);
	int rc = ofi_amd_tuner_query(&q, 1, out);
	if (rc == 0) {
		if (ctx->memo.size() > (1u << 20)) {
			ctx->memo.clear(); /* bounded memory for adversarial size streams */
		}
		ctx->memo.emplace(key, *out);
	}
	return rc;
}

/* nccl_ofi_tuner_get_coll_info(_v6), :162-182 / :199-217 */
ncclResult_t tuner_get_coll_info(void *context, ncclFunc_t collType, size_t nBytes, int numPipeOps,
				 float **collCostTable, int numAlgo, int numProto, int *nChannels)
{
	auto *ctx = static_cast<tuner_ctx *>(context);
	if (!ctx || (int)collType < 0 || (int)collType >= NCCL_NUM_FUNCTIONS || !collCostTable ||
	    ctx->nodes == 0 || ctx->ranks == 0) {
		return ncclSuccess; /* fall back to NCCL's tuner */
	}
	float(*table)[NCCL_NUM_PROTOCOLS] = (float(*)[NCCL_NUM_PROTOCOLS])collCostTable;
	uint32_t mask = kAllAllowed;
	if (!ctx->model) {
		/* regions whose cell NCCL marked as ignored, or that this NCCL does not know, are
		 * skipped (src/tuner/nccl_ofi_regions.cpp:2109-2114) */
		mask = 0;
		for (int a = 0; a < NCCL_NUM_ALGORITHMS && a < numAlgo; a++) {
			for (int p = 0; p < NCCL_NUM_PROTOCOLS && p < numProto; p++) {
				if (table[a][p] != (float)NCCL_ALGO_PROTO_IGNORE) {
					mask |= 1u << (a * NCCL_NUM_PROTOCOLS + p);
				}
			}
		}
	}
	ofi_amd_tuner_answer_t ans;
	int rc = ask(ctx, ctx->model, (int)collType, nBytes, ctx->model ? numPipeOps : 0, mask, 0, 0, &ans);
	if (rc != 0) {
		/* the cost table is left as NCCL filled it: its own tuner decides this collective */
		TUNER_WARN("GPU tuner query failed (%d): falling back to NCCL's tuner for this call", rc);
		return ncclSuccess;
	}
	if (ans.algo >= 0 && ans.algo < numAlgo && ans.proto >= 0 && ans.proto < numProto) {
		table[ans.algo][ans.proto] = 0.0f;
		if (ans.nchannels >= 0 && nChannels) {
			*nChannels = ans.nchannels;
		}
	}
	return ncclSuccess;
}

ncclResult_t tuner_get_coll_info_v6(void *context, ncclFunc_t collType, size_t nBytes, int numPipeOps,
				    float **collCostTable, int numAlgo, int numProto, int /* regBuff */,
				    int *nChannels)
{
	return tuner_get_coll_info(context, collType, nBytes, numPipeOps, collCostTable, numAlgo, numProto,
				   nChannels);
}

/* nccl_ofi_tuner_get_coll_info_v2, :246-271 */
ncclResult_t tuner_get_coll_info_v2(void *context, ncclFunc_t collType, size_t nBytes, int /* collNet */,
				    int nvlsSupport, int numPipeOps, int *algorithm, int *protocol,
				    int * /* nChannels */)
{
	auto *ctx = static_cast<tuner_ctx *>(context);
	if (!ctx || (int)collType < 0 || (int)collType >= NCCL_NUM_FUNCTIONS || ctx->nodes == 0 ||
	    ctx->ranks == 0) {
		return ncclSuccess;
	}
	uint32_t mask = kAllAllowed;
	if (!nvlsSupport) {
		mask &= ~(7u << (kAlgoNvlsTree * NCCL_NUM_PROTOCOLS));
	}
	if (!ctx->model) {
		mask &= ~(7u << (kAlgoPat * NCCL_NUM_PROTOCOLS)); /* PAT is not expressible in v2 */
	}
	ofi_amd_tuner_answer_t ans;
	int rc = ask(ctx, ctx->model, (int)collType, nBytes, ctx->model ? numPipeOps : 0, mask, 0, 0, &ans);
	if (rc != 0) {
		TUNER_WARN("GPU tuner query failed (%d): falling back to NCCL's tuner for this call", rc);
		return ncclSuccess;
	}
	if (ans.algo >= 0 && algorithm && protocol) {
		*algorithm = ans.algo;
		*protocol = ans.proto;
	}
	return ncclSuccess;
}

/* nccl_ofi_tuner_get_chunk_size, :224-239: only the region tuner has an opinion */
ncclResult_t tuner_get_chunk_size(void *context, ncclFunc_t collType, size_t nBytes, int algo, int proto,
				  int /* nChannels */, size_t *chunkSize)
{
	auto *ctx = static_cast<tuner_ctx *>(context);
	if (!ctx || ctx->model || !chunkSize || algo < 0 || algo >= NCCL_NUM_ALGORITHMS || proto < 0 ||
	    proto >= NCCL_NUM_PROTOCOLS || (int)collType < 0 || ctx->nodes == 0 || ctx->ranks == 0) {
		return ncclSuccess;
	}
	ofi_amd_tuner_answer_t ans;
	int rc = ask(ctx, 2, (int)collType, nBytes, 0, kAllAllowed, algo, proto, &ans);
	if (rc != 0) {
		TUNER_WARN("GPU tuner query failed (%d): chunk size left to NCCL", rc);
		return ncclSuccess;
	}
	if (ans.chunk_size != 0) {
		*chunkSize = (size_t)ans.chunk_size;
	}
	return ncclSuccess;
}

} // namespace

extern "C" {

int ofi_amd_tuner_ctx_stats(const void *context, ofi_amd_tuner_ctx_stats_t *out)
{
	auto *ctx = static_cast<const tuner_ctx *>(context);
	if (!ctx || !out || ctx->magic != kCtxMagic) {
		return -EINVAL;
	}
	std::lock_guard<std::mutex> g(const_cast<tuner_ctx *>(ctx)->lock);
	*out = ctx->stats;
	return 0;
}

__attribute__((visibility("default"))) ncclTuner_v3_t ncclTunerPlugin_v3 = {
	"nccl_ofi_tuner", tuner_init, tuner_get_coll_info, tuner_destroy
};

__attribute__((visibility("default"))) ncclTuner_v6_t ncclTunerPlugin_v6 = {
	"nccl_ofi_tuner", tuner_init_v6, tuner_get_coll_info_v6, tuner_destroy, tuner_get_chunk_size
};

__attribute__((visibility("default"))) ncclTuner_v2_t ncclTunerPlugin_v2 = {
	"nccl_ofi_tuner", tuner_init_v2, tuner_get_coll_info_v2, tuner_destroy
};

} /* extern "C" */
