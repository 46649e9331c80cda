# 1/ln(2) as the nearest fp32 (0x3FB8AA3B): gates are accumulated in log2 units so that the
# kernels can use exp2 (fla/ops/utils/constant.py:10).  The HIP kernels hard-code the same value.
RCP_LN2 = 1.4426950216
