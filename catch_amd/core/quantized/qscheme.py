"""Default calibration options (counterpart of torch_mlu/core/quantized/qscheme.py:11-19).

  iteration    number of calibration batches an observer accepts
  use_avg      running mean of the per-batch min/max instead of the extreme values
  data_scale   factor applied to each batch's min/max
  mean, std    first-conv normalisation (values in [0,1]; stored x255)
  firstconv    fold (x-mean)/std in front of the first convolution
  per_channel  one weight scale per output channel
"""
mlu_qscheme = {
    "iteration": 1,
    "use_avg": False,
    "data_scale": 1.0,
    "mean": [0, 0, 0],
    "std": [1, 1, 1],
    "firstconv": True,
    "per_channel": False,
}
