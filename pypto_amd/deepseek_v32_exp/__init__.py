"""Drop-in operator modules for the reference's models/deepseek_v32_exp directory.

The reference's drivers import the operator modules by bare name
(models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:19-24); add this directory to
``sys.path`` (or import ``pypto_amd.deepseek_v32_exp.<module>``) to get the same names.
"""
