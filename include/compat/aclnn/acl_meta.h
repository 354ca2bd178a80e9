/* Takes the place of <aclnn/acl_meta.h> (the reference's stand-in: mock/include/aclnn/acl_meta.h). */
#ifndef MOE_KV_HIP_COMPAT_ACLNN_ACL_META_H_
#define MOE_KV_HIP_COMPAT_ACLNN_ACL_META_H_
#include "../../aclnn_hip.h"
#endif
