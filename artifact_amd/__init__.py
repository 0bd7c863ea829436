"""MI355X-native reuse-aware GNN neighbour aggregation (drop-in for the ROF operator path).

Modules: `reuse_search_ext` (CPU plan builder, upstream module of the same name), `ROF` (operator
boundary, upstream extension of the same name), `reuse_conv` (layer API), `layout` (device layout),
`graphgen` (synthetic inputs).  The compute path lives in librof.so (csrc/), built by
`python -m artifact_amd.build`; nothing falls back to the CPU when it is missing.
"""
__version__ = "0.1.0"
