"""MI355X (gfx950) implementation of the MoR fake-quantization path.

`mor_amd._cabi` binds the C ABI of libmor_hip.so (include/mor_hip.h); `mor_amd.ops` registers the `torch.ops.mor.*`
operators on top of it and mirrors the reference's `mor.ops` Python API.  `import mor` gives the drop-in name.
`mor_amd.wire` adds what the reference has no op for: the MX wire format (codes + E8M0 scale bytes);
`mor_amd.batch` runs fake_quantize over a list of tensors in one call.
"""
from . import _cabi  # noqa: F401
from . import ops  # noqa: F401
from . import wire  # noqa: F401
from . import stats  # noqa: F401
from . import batch  # noqa: F401

__all__ = ["ops", "wire", "stats", "batch"]
