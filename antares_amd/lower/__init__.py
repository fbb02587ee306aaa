"""Lowering of parsed programs to gfx950 kernels: generic templates and the
table of hand-written kernels that take over known operator patterns."""
from .hip_codegen import contraction_slices, lower_graph, lower_statement, KernelPlan
