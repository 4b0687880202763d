/*
 * Negative errno -> ncclResult_t, as the reference's entry points do it
 * (nccl_net_ofi_retval_translate, include/nccl_ofi_api.h:30-75).
 */
#ifndef OFI_AMD_NCCL_TRANSLATE_HPP_
#define OFI_AMD_NCCL_TRANSLATE_HPP_

#include <cerrno>

#include "ofi_amd_nccl_err.h"

namespace ofi_amd {

inline ncclResult_t nccl_result_of(int rc)
{
	switch (rc) {
	case 0:
		return ncclSuccess;
	case -EINVAL:
		return ncclInternalError; /* "invalid arguments to plugin calls should return ncclInternalError" */
	case -EMSGSIZE:
		return ncclInvalidUsage;
	case -ECONNABORTED:
	case -ECONNRESET:
	case -ECONNREFUSED:
	case -ENOTCONN:
	case -EHOSTDOWN:
	case -EHOSTUNREACH:
		return ncclRemoteError;
	default:
		return ncclSystemError;
	}
}

} // namespace ofi_amd

#endif
