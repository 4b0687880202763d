/*
 * The slice of the NCCL / RCCL external tuner ABI this library implements, restated:
 * result codes (nccl/err.h), logger callback (nccl/net.h:40-43), collective /
 * algorithm / protocol numbering (nccl/tuner.h:14-44) and the three plugin structs
 * NCCL looks up by symbol name -- ncclTuner_v2_t (nccl/tuner_v2.h), ncclTuner_v3_t
 * (nccl/tuner.h:46-87) and ncclTuner_v6_t (nccl/tuner_v6.h:19-82).  Field order and
 * function signatures are the contract; everything else NCCL passes is opaque here.
 */
#ifndef OFI_AMD_NCCL_TUNER_ABI_H_
#define OFI_AMD_NCCL_TUNER_ABI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
	ncclSuccess = 0,
	ncclUnhandledCudaError = 1,
	ncclSystemError = 2,
	ncclInternalError = 3,
	ncclInvalidArgument = 4,
	ncclInvalidUsage = 5,
	ncclRemoteError = 6
} ncclResult_t;

typedef enum {
	NCCL_LOG_NONE = 0, NCCL_LOG_VERSION = 1, NCCL_LOG_WARN = 2, NCCL_LOG_INFO = 3,
	NCCL_LOG_ABORT = 4, NCCL_LOG_TRACE = 5
} ncclDebugLogLevel;
enum { NCCL_INIT = 1, NCCL_TUNING = 64 };
typedef void (*ncclDebugLogger_t)(ncclDebugLogLevel level, unsigned long flags, const char *file,
				  int line, const char *fmt, ...);

typedef enum {
	ncclFuncBroadcast = 0, ncclFuncReduce = 1, ncclFuncAllGather = 2, ncclFuncReduceScatter = 3,
	ncclFuncAllReduce = 4, ncclFuncSendRecv = 5, ncclFuncSend = 6, ncclFuncRecv = 7, ncclNumFuncs = 8
} ncclFunc_t;

#define NCCL_NUM_FUNCTIONS 5
#define NCCL_NUM_ALGORITHMS 7
#define NCCL_NUM_PROTOCOLS 3
#define NCCL_ALGO_PROTO_IGNORE -1.0

/* opaque to this plugin: only pointers to them cross the boundary */
typedef struct ncclTunerConstants_v6 ncclTunerConstants_v6_t;
typedef struct ncclNvlDomainInfo_v6 ncclNvlDomainInfo_v6_t;

typedef struct {
	const char *name;
	ncclResult_t (*init)(size_t nRanks, size_t nNodes, ncclDebugLogger_t logFunction, void **context);
	ncclResult_t (*getCollInfo)(void *context, ncclFunc_t collType, size_t nBytes, int collNetSupport,
				    int nvlsSupport, int numPipeOps, int *algorithm, int *protocol,
				    int *nChannels);
	ncclResult_t (*destroy)(void *context);
} ncclTuner_v2_t;

typedef struct {
	const char *name;
	ncclResult_t (*init)(size_t nRanks, size_t nNodes, ncclDebugLogger_t logFunction, void **context);
	ncclResult_t (*getCollInfo)(void *context, ncclFunc_t collType, size_t nBytes, int numPipeOps,
				    float **collCostTable, int numAlgo, int numProto, int *nChannels);
	ncclResult_t (*destroy)(void *context);
} ncclTuner_v3_t;

typedef struct {
	const char *name;
	ncclResult_t (*init)(void **ctx, uint64_t commId, size_t nRanks, size_t nNodes,
			     ncclDebugLogger_t logFunction, ncclNvlDomainInfo_v6_t *nvlDomainInfo,
			     ncclTunerConstants_v6_t *constants);
	ncclResult_t (*getCollInfo)(void *context, ncclFunc_t collType, size_t nBytes, int numPipeOps,
				    float **collCostTable, int numAlgo, int numProto, int regBuff,
				    int *nChannels);
	ncclResult_t (*finalize)(void *context);
	ncclResult_t (*getChunkSize)(void *context, ncclFunc_t collType, size_t nBytes, int algo, int proto,
				     int nChannels, size_t *chunkSize);
} ncclTuner_v6_t;

extern ncclTuner_v2_t ncclTunerPlugin_v2;
extern ncclTuner_v3_t ncclTunerPlugin_v3;
extern ncclTuner_v6_t ncclTunerPlugin_v6;

#ifdef __cplusplus
}
#endif
#endif
