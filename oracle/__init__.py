"""CPU oracle for the quantized DeepSeek-V3.2 sparse-attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is the checker used by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py``.  The product path is the HIP
library under ``pypto_amd/csrc`` and fails loudly when that library is absent.

Contents
--------
``sfa_oracle``   restatement of the sparse-flash-attention torch goldens
                 (reference: examples/models/deepseek_v32_exp/
                 deepseekv32_sparse_flash_attention_quant.py:49-254).
``li_oracle``    restatement of the lightning-indexer torch golden
                 (reference: examples/models/deepseek_v32_exp/
                 deepseekv32_lightning_indexer_quant.py:184-269) with the
                 canonical, fully specified arithmetic and tie rule.
``oracle_c.c``   the same two algorithms in plain scalar C with hand-written
                 bf16/fp16 rounding; an independent second statement used to
                 cross-check the Python one and as the timed CPU baseline.

Pinning status (which independent check pins which function) is listed in the
header of each module.
"""
