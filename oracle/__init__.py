"""CPU oracle (test infrastructure): ctypes bindings of libiris_oracle.so,
libiris_cpu_baseline.so and, when it has been built, _ref/libiris_ref.so.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this package. The product (iris_c_amd) never does.
"""
from .binding import (  # noqa: F401
    Oracle, CpuBaseline, Reference, oracle, cpu_baseline, reference, build,
    f32_to_bf16, bf16_to_f32,
)
