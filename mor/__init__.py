"""Drop-in name of the reference package: `import mor; mor.ops.fake_quantize(...)` (mor/__init__.py:1-2)."""
import torch  # noqa: F401
from mor_amd import _cabi as _C  # noqa: F401
from mor_amd import ops  # noqa: F401
