# Added to a block's absmax before the GELU-forward scale is formed (reference: Jetfire/Nonlinear/common.py:3).
SCALE_MIN_THRES = 5e-5
