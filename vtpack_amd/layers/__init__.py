from .dge import DynamicGrainedEncoder, DynamicRouter
from .grained_sample import (
    grained_sample_compress,
    grained_sample_compress_dense,
    grained_sample_decompress,
    grained_sample_decompress_dense,
    grained_sample_index_to_patch,
    grained_sample_index_to_patch_dense,
)
from .sparse_ops import (
    batched_sparse_gemm,
    batched_sparse_attention,
)
