"""gpu_rsfk -- RSFK K-NN-graph construction on AMD MI355X (gfx950).

Same public names as the reference package (``from .RSFK import RSFK, test``).
"""
from .RSFK import RSFK, ForestLog, random_motion, test  # noqa: F401
from .graph import symmetric_knn_graph  # noqa: F401
