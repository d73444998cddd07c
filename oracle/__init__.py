"""CPU oracle for the DiT attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: it is the checker used by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py``.  The product path
(``maxdiffusion_amd``) runs hand-written HIP kernels and raises when its
shared library is missing; it never falls back to anything in here.

Every function restates, in numpy, the arithmetic of the reference file:line it
cites (paths relative to ``src/maxdiffusion/`` of AI-Hypercomputer/maxdiffusion).
"""
from .dit_attention import *  # noqa: F401,F403
from .inputs import *  # noqa: F401,F403
