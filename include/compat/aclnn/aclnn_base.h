/* Takes the place of <aclnn/aclnn_base.h> (the reference's stand-in: mock/include/aclnn/aclnn_base.h). */
#ifndef MOE_KV_HIP_COMPAT_ACLNN_ACLNN_BASE_H_
#define MOE_KV_HIP_COMPAT_ACLNN_ACLNN_BASE_H_
#include "../../aclnn_hip.h"
#endif
