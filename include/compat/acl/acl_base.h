/* Takes the place of <acl/acl_base.h> (the reference's stand-in: mock/include/acl/acl_base.h). */
#ifndef MOE_KV_HIP_COMPAT_ACL_ACL_BASE_H_
#define MOE_KV_HIP_COMPAT_ACL_ACL_BASE_H_
#include "../../aclnn_hip.h"
#endif
