"""The hot-path operator catalog: each a declared class over one hand-written HIP kernel."""

from .copy import Copy
from .elementwise_add import ElementwiseAdd, RowwiseAdd
from .elementwise_mul import ElementwiseMul, RowwiseMul
from .gemm import GEMM
from .gemv import GEMV
from .mha import MHA
from .rms_norm import RMSNorm
from .rope import RoPE
from .sample import Sample
from .silu import SiLU

__all__ = ["Copy", "ElementwiseAdd", "ElementwiseMul", "GEMM", "GEMV", "MHA", "RMSNorm", "RoPE", "RowwiseAdd",
           "RowwiseMul", "Sample", "SiLU"]

#: Every operator by its class name (iron/operators/__init__.py:69-72).
CATALOG = {name: globals()[name] for name in __all__}
