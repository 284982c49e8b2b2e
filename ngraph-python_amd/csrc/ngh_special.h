// Hand-specialised kernels for the fused patterns that dominate training
// graphs.  Each entry recognises one op program (by structure, not by
// pointer values) and runs it with registers in VGPRs instead of through the
// interpreter.  Filled in below; an empty table means every stage goes
// through the interpreter.
#pragma once
#include "ngh_device.h"

namespace ngh {

inline const char* special_name(int) { return "none"; }
inline int match_special(int /*family*/, int /*V*/, const KArgs& /*k*/, long long /*tail*/) { return -1; }
inline hipError_t launch_special(int, hipStream_t, int, const KArgs&, unsigned, unsigned) {
    return hipErrorInvalidValue;
}

}  // namespace ngh
