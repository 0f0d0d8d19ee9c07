from torchrec_amd.sparse.jagged_tensor import (  # noqa: F401
    JaggedTensor,
    KeyedJaggedTensor,
    KeyedTensor,
)
