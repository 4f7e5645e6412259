"""``ttnn.experimental``: entry points that tt-metal does not have under these names, for callers that want fewer launches."""
from __future__ import annotations

from .matmul import gated_linear  # noqa: F401
