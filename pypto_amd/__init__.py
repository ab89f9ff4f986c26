"""pypto_amd -- MI355X (gfx950) implementation of the quantized DeepSeek-V3.2 sparse-attention path.

Operators (same names and signatures as the reference examples they replace):

* :func:`sparse_flash_attention_quant_d` / :func:`sparse_flash_attention_quant_p`
* :func:`sparse_attention_antiquant_d` / :func:`sparse_attention_antiquant_p` (packed 656-byte cache rows)
* :func:`lightning_indexer_decode`
* :func:`lightning_indexer_prolog_quant` (the projection stage in front of the indexer)
* :func:`mla_prolog_quant_d` / :func:`mla_prolog_quant_p` (the projection stage in front of the attention)
* :func:`mla_indexer_prolog_quant_d` / :func:`mla_indexer_prolog_quant_p` (both prologs in one call)

plus :func:`from_torch`, the tensor hand-over of the reference's jit convention.  The computation
runs in hand-written HIP kernels behind a C ABI (``include/pypto_amd_sfa.h``); there is no CPU
fallback.
"""
from .converter import Tensor, from_torch  # noqa: F401
from .lightning_indexer_quant_impl import LightningIndexerConfigs, lightning_indexer_decode  # noqa: F401
from .lightning_indexer_prolog_quant_impl import (IndexerPrologQuantAttr, IndexerPrologQuantConfigs,  # noqa: F401
                                                  IndexerPrologQuantInput, IndexerPrologQuantOutput,
                                                  lightning_indexer_prolog_quant)
from .mla_indexer_prolog_quant_impl import mla_indexer_prolog_quant_d, mla_indexer_prolog_quant_p  # noqa: F401
from .mla_prolog_quant_impl import (MlaQuantInputs, MlaTileConfig, RopeTileShapeConfig,  # noqa: F401
                                    mla_prolog_quant_d, mla_prolog_quant_p)
from .sparse_attention_antiquant_impl import sparse_attention_antiquant_d, sparse_attention_antiquant_p  # noqa: F401
from .sparse_flash_attention_quant_impl import (SaTileShapeConfig, sparse_flash_attention_quant_d,  # noqa: F401
                                                sparse_flash_attention_quant_p)

__version__ = "0.6.0"
