#!/usr/bin/env python3
"""`python setup.py build_ext --inplace` -- the build command the reference documents
(README.md:16-18, setup.py:76-96) -- forwarded to build.py, which drives hipcc for gfx950
directly (no CUDAExtension, no hipify pass).  Any other command is refused."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

import build  # noqa: E402

if __name__ == "__main__":
    if len(sys.argv) >= 2 and sys.argv[1] == "build_ext":
        sys.exit(build.main([]))
    sys.stderr.write("only `python setup.py build_ext --inplace` is supported; see build.py\n")
    sys.exit(2)
