/* Takes the place of <acl/acl.h> (CANN; the reference's stand-in: mock/include/acl/acl.h) when the
 * engine is built against libmoe_kv_hip.so: the declarations live in aclnn_hip.h. */
#ifndef MOE_KV_HIP_COMPAT_ACL_ACL_H_
#define MOE_KV_HIP_COMPAT_ACL_ACL_H_
#include "../../aclnn_hip.h"
#endif
