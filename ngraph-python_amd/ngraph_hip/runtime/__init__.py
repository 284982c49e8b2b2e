from ngraph_hip.runtime.hiplib import (  # noqa: F401
    HipLibraryError, HipRuntime, DryRunRuntime, FusedSpecBuilder, load_library, library_path, OPCODES,
    NGH_F32, NGH_FLEX16, NGH_I32, NGH_F16, NGH_U32, NGH_I16, NGH_I8, NGH_U8)
