// Shared by the two halves of the C ABI (the thin kernel ABI and the aclnn-compatible
// operator shim): status reporting and small helpers.
#pragma once

#include <string>

#include "mlakv.h"

namespace mlakv_abi {

// Records printf-style text as the calling thread's last error and returns `code`.
mlakvStatus Fail(mlakvStatus code, const char* format, ...) __attribute__((format(printf, 2, 3)));
mlakvStatus FailText(mlakvStatus code, const std::string& text);
const char* LastError();
// Compute units of the current device; 256 when no device is visible (plan arithmetic only).
int ComputeUnits();

}  // namespace mlakv_abi
