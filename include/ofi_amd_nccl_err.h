/*
 * ncclResult_t as NCCL's plugin headers define it (3rd-party/nccl/cuda/include/nccl/err.h:9-16
 * in the reference), under the same include guard, so that this library's headers and NCCL's can
 * be included together in either order.  Plain C.
 */
#ifndef OFI_AMD_NCCL_ERR_H_
#define OFI_AMD_NCCL_ERR_H_

#ifndef NCCL_ERR_H_
#define NCCL_ERR_H_
typedef enum { ncclSuccess                 =  0,
               ncclUnhandledCudaError      =  1,
               ncclSystemError             =  2,
               ncclInternalError           =  3,
               ncclInvalidArgument         =  4,
               ncclInvalidUsage            =  5,
               ncclRemoteError             =  6 } ncclResult_t;
#endif

#endif /* OFI_AMD_NCCL_ERR_H_ */
