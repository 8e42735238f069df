"""Switches of the reference's kernel package (flex_gemm/kernels/triton/spconv/config.py:7-8), kept so that code which
sets them keeps running (tests/submconv/train_benchmark.py:135 does).

allow_tf32: gfx950 has no TF32 matrix instruction; float32 inputs are multiplied on the FP32 MFMA path whatever this
says, so the flag changes nothing (the reference defaults it to False on ROCm as well).
USE_ON_THE_FLY_WEIGHT_TRANSPOSE: the input-gradient pass always reads a weight panel repacked for it; nothing to choose.
There is no autotune_config: tile shapes come from the library's fixed schedule table (fgx_table_lookup)."""

allow_tf32 = False
USE_ON_THE_FLY_WEIGHT_TRANSPOSE = True
