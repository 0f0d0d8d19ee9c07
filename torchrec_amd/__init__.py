"""torchrec_amd — MI355X-native quantized embedding inference.

Drop-in for the quantized inference path of TorchRec
(``torchrec.quant.EmbeddingBagCollection`` / ``EmbeddingCollection`` over a
``KeyedJaggedTensor``), executed by hand-written gfx950 HIP kernels behind the
C ABI in ``include/torchrec_amd.h``.
"""
from torchrec_amd.sparse.jagged_tensor import JaggedTensor, KeyedJaggedTensor, KeyedTensor  # noqa: F401
from torchrec_amd.types import DataType  # noqa: F401

__version__ = "0.1.0"
