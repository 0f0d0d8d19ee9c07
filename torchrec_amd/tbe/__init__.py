from torchrec_amd.tbe.enums import EmbeddingLocation, PoolingMode, SparseType  # noqa: F401
