from torchrec_amd.tbe.enums import EmbeddingLocation, PoolingMode, SparseType  # noqa: F401
from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import (  # noqa: F401,E402
    ROW_PADDING_BUDGET_BYTES,
    get_default_row_padding,
    line_padded_row_stride,
    set_default_row_padding,
)
