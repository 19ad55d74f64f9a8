"""CPU checker for the HIP library — TEST INFRASTRUCTURE ONLY.

`oracle` restates the reference's arithmetic for the sparse-retrieval / KV-transfer path on
the CPU.  Only tests, the smoke check and the benchmark's CPU-baseline leg may import it;
the shipped package never does.

Two layers:
  * `oracle.c_api`  — ctypes bindings of libucm_oracle.so (ucm_oracle.c, plain C);
  * `oracle.brute`  — independent numpy / pure-Python restatements for tiny inputs, used to
                      pin the C code itself.
`oracle.ref_backend()` loads the reference's own CPU retrieval backend when it has been
compiled into oracle/_ref/ (see the Makefile); it returns None otherwise.
"""
from . import brute, c_api  # noqa: F401
from .c_api import ref_backend  # noqa: F401
