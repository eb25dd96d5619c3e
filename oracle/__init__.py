"""CPU oracle for the DeepSeek-V3.2 quantized decode-attention path and the two GLM-4.5 operators beside it.

TEST INFRASTRUCTURE ONLY.  Nothing under ``pypto_amd/`` imports this package.
It may be imported from ``tests/``, from ``__graft_entry__.smoke()`` and from
the ``cpu_baseline`` leg of ``bench.py`` - always as the checker or the timed
CPU baseline, never as a code path of the product.

The modules restate, in plain torch/numpy on the CPU, the torch goldens that
the reference keeps inside its operator drivers (paths relative to the
reference checkout):

  paged.py    page-table index math            python/pypto/experimental/gather.py:27-82
                                               models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:262-300
  sfa.py      sparse flash attention goldens   models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:54-259
                                               models/deepseek_v32_exp/deepseekv32_sparse_attention_antiquant.py:54-141,359-457
  indexer.py  lightning indexer golden         models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:46-307
  topk.py     top-k ordering rule              framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494,2734-2749
  compare.py  tolerance comparators            models/deepseek_v32_exp/utils/compare.py:16-125
  indexer_prolog.py  lightning-indexer prolog  models/deepseek_v32_exp/deepseekv32_lightning_indexer_prolog_quant.py:30-288
  mla_prolog.py      MLA prolog (int8 form) and the fused MLA + indexer prolog  models/deepseek_v32_exp/deepseekv32_mla_prolog_quant.py:32-441, deepseekv32_mla_indexer_prolog_quant.py:336-393,711-713
  select_experts.py  grouped expert selection  models/glm_v4_5/glm_select_experts.py:274-313
                                               python/tests/ut/interpreter/_ops/moe_gating_topk.py:223-287
  gqa.py      paged GQA decode goldens         models/glm_v4_5/glm_attention.py:1374-1483
                                               models/glm_v4_5/utils/golden/attn_golden.py:97-130,300-321
  attention_pre_quant.py  GLM attention prolog models/glm_v4_5/glm_attention_pre_quant.py:133-231,235-505,591-619

The arithmetic of those goldens is PyTorch's CPU arithmetic (an unpinned,
un-vendored dependency of the reference), so every function here is pinned in
``tests/test_oracle_*.py`` against the known answers the reference holds
(doc-string examples, deterministic test buffers), against closed forms
(IEEE round-to-nearest-even conversions done by hand in integer arithmetic,
float64 textbook attention, brute-force integer dot products) and against
invariants.  Parity unpinned: two steps of ``attention_pre_quant.py`` (``quantize`` and the int8 projection's
dequantisation), which the reference's golden delegates to NPU library calls whose outputs it holds no fixture of - that
module's header says what they follow instead.  No other function is left unpinned.
"""
