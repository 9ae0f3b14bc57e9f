"""Modules with the names and call signatures of the reference's three compiled extension modules
(`clustenqk_cuda`, `clustenav_cuda`, `clustenwf_cuda`; clusten/clusten.py:9-11 imports them), bound to
libclusten_hip.so through its C ABI.  For a maintainer who keeps the reference's own clusten/clusten.py:
`from clusten_ext import clustenqk_cuda, clustenav_cuda, clustenwf_cuda` in place of the compiled modules."""
from . import clustenav_cuda, clustenqk_cuda, clustenwf_cuda  # noqa: F401
