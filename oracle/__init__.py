"""CPU oracle for the quantized-linear forward path.

TEST INFRASTRUCTURE ONLY: the checker the HIP kernels are compared against.
Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this package; nothing under ``neuropress_amd`` does.

Two layers:

* ``np_oracle.c`` (built by ``make -C oracle`` into ``libnp_oracle.so``) -- the
  scalar C restatement of the reference algorithm, bound here through ctypes
  on numpy arrays.
* ``torch_path`` -- the reference's CPU forward (unpack -> gather -> F.linear)
  restated with torch ops, used for the timed CPU baseline.
"""

from .oracle import (  # noqa: F401
    DT_BF16,
    DT_F16,
    DT_F32,
    bits_for,
    build,
    linear_f64,
    pack_indices,
    q_decode,
    rvq_decode,
    unpack_indices,
    vq_decode,
)
