"""Constants of the kernel library's C header, read from its text: the header is the one place
where they are written, and reading it needs neither a GPU nor a built library."""
from __future__ import annotations

import os
import re

_HEADER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sb_hip.h")


def define(name: str) -> int:
    """The integer that ``#define name`` of sb_hip.h gives."""
    with open(_HEADER) as f:
        m = re.search(rf"^#define\s+{re.escape(name)}\s+(-?\d+)\s*$", f.read(), re.MULTILINE)
    if m is None:
        raise RuntimeError(f"{_HEADER} defines no integer {name}")
    return int(m.group(1))


PAGE = define("SB_PAGE")          # tokens per cache page
