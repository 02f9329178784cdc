"""The operator catalog: the hot path's operators and the sibling decoders', each a declared class over one
hand-written HIP kernel."""

from .axpy import AXPY
from .clamp import Clamp
from .copy import Copy, Gather, GatherWords
from .elementwise_add import ElementwiseAdd, RowwiseAdd
from .elementwise_mul import ElementwiseMul, RowwiseMul
from .gelu import GELU
from .gemm import GEMM
from .gemv import GEMV
from .layer_norm import LayerNorm
from .mha import MHA
from .relu import ReLU
from .rms_norm import RMSNorm
from .rope import RoPE
from .sample import Sample
from .sigmoid import Sigmoid
from .silu import SiLU
from .softmax import Softmax
from .tanh import Tanh

__all__ = ["AXPY", "Clamp", "Copy", "ElementwiseAdd", "ElementwiseMul", "GELU", "GEMM", "GEMV", "Gather", "GatherWords",
           "LayerNorm", "MHA",
           "RMSNorm", "ReLU", "RoPE", "RowwiseAdd", "RowwiseMul", "Sample", "Sigmoid", "SiLU", "Softmax", "Tanh"]

#: Every operator by its class name (iron/operators/__init__.py:69-72).
CATALOG = {name: globals()[name] for name in __all__}
