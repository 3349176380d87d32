import math

import numpy as np
import torch.nn as nn


def glorot_uniform_af(x, gain=1.0):
    """Xavier-uniform with fans taken from the last two dims (times the receptive field of the
    leading dims) - the initialiser of the reference's fastnn Linear
    (fastfold/model/fastnn/initializer.py:7-29)."""
    fan_in, fan_out = x.shape[-2:]
    if x.dim() > 2:
        rf = int(np.prod(x.shape[:-2]))
        fan_in, fan_out = fan_in * rf, fan_out * rf
    bound = math.sqrt(3.0) * gain * math.sqrt(2.0 / float(fan_in + fan_out))
    nn.init.uniform_(x, -bound, bound)
    return x
