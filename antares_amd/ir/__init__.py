"""einstein_v2 front-end: text IR -> typed statements -> Graph."""
from .nodes import Expr, const, cast, merge_dtype, C_TYPES, ITEMSIZE, walk, rewrite
from .parser import IRSyntaxError, Statement, TensorInfo, parse_statement, parse_tensor_spec, split_statements
from .graph import Graph, parse_program, fuse_elementwise, split_wide_reductions, bake_small_reduce_extents, pad_guarded_factors
from .printer import to_ir, statement_to_ir, canonical
