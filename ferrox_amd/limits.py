"""Sizes the kernels take, in one place: the typed configurations refuse a model beyond them
when config.json is read, the parts when they are built, and the kernels' entry points once
more at the call (the constants of the same names in csrc/)."""

MOE_MAX_EXPERTS = 1024      # E_MAX in csrc/moe.hip: a token's scores live in LDS
MOE_MAX_TOP_K = 32          # K_MAX in csrc/moe.hip: a lane per selection
HEAD_DIM_STEP = 16          # the MFMA attention reads 16 columns of a head at a time
HEAD_DIM_MAX = 256          # HD_MAX in csrc/attention.hip
