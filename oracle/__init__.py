"""CPU oracle for the quantized-KV attention path -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this package; the shipped library never does.  `oracle.hs_oracle` wraps the C
restatement (libhs_oracle.so, built by `python oracle/build.py`), and
`oracle.deltanet_chunked` / `oracle.reference_path` restate the reference's
tensor-op sequences with numpy / libtorch CPU ops.
"""
from .hs_oracle import *  # noqa: F401,F403
