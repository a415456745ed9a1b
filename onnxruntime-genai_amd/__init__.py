"""MI355X-native search & sampling backend (HIP kernels behind a C ABI).

The directory name contains a hyphen, so load it with `load_package()` from
`__graft_entry__.py` (it registers the package as `onnxruntime_genai_amd`)."""
from .capi import (SearchContext, LogitsXform, SampleParams, BeamScorer, load_library, library_path,  # noqa: F401
                   MI355X_F32, MI355X_F16)
