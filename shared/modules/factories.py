"""`shared.modules.factories` of the reference, served by pam_amd.factories (same function names,
description formats and keyword filtering, shared/modules/factories.py:103-298)."""
from pam_amd.factories import *        # noqa: F401,F403
from pam_amd.factories import (CustomConv2d, CustomLinear, Bias, Gain, LazyBias, LazyGain, call_valid_kwargs,   # noqa: F401
                               get_activation_factory, get_bias_factory, get_conv_factory, get_function_dict, get_gain_factory,
                               get_linear_factory, get_module_factory, get_norm_factory, get_sequential_factory, get_valid_kwargs)
