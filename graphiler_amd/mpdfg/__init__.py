"""Compiler front end: user-defined message / reduce / update functions ->
one TorchScript plan of ``my_ops::*`` graph operators (the reference's
python/graphiler/{mpdfg_builder,mpdfg_optimizer,update_all,dgl_udf_batch}.py over
src/builder and src/optimizer), rebuilt on TorchScript's Python graph API.
"""
from .batch import EdgeBatchDummy, NodeBatchDummy  # noqa: F401
from .builder import MPDFG, BuildError, mpdfg_builder  # noqa: F401
from .passes import dedup, fusion, optimize, reorder, split  # noqa: F401
from .runtime import GraphData, update_all  # noqa: F401
