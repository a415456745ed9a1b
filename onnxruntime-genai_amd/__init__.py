"""MI355X-native search & sampling backend (HIP kernels behind a C ABI).

The directory name contains a hyphen, so load it with `load_package()` from
`__graft_entry__.py` (it registers the package as `onnxruntime_genai_amd`)."""
from .capi import (SearchContext, LogitsXform, SampleParams, BeamScorer, argmax_static, load_library,  # noqa: F401
                   library_path,
                   MI355X_F32, MI355X_F16)
