/* <acl/acl.h> under the name that the reference's kernel and host sources include: the Ascend runtime calls they make,
 * expressed on the HIP runtime (pto/host/acl_hip.h). */
#ifndef PTO_ACL_ACL_H
#define PTO_ACL_ACL_H
#include "pto/host/acl_hip.h"
#endif
