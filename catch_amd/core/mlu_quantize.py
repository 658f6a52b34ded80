"""Module-swap quantization tool (counterpart of torch_mlu/core/mlu_quantize.py:155-230).

    calib = quantize_dynamic_mlu(model, {'per_channel': True, 'firstconv': False}, dtype='int8', gen_quant=True)
    calib(x_cpu)                                  # float pass, observers record min/max
    ckpt = calib.state_dict()                     # + scale / quantized_mode / ...
    qmodel = quantize_dynamic_mlu(model)          # swap only
    qmodel.load_state_dict(ckpt); qmodel.to('cuda')(x_gpu)   # torch_mlu::conv2d / linear
"""
import copy

import torch.nn as nn

from .quantized.default_mappings import DEFAULT_MLU_MODULE_MAPPING, DEFAULT_QCONFIG_PROPAGATE_WHITE_LIST
from .quantized.observer import (mlu_activation_observer_dict, mlu_weight_observer,
                                 mlu_weight_per_channel_observer)
from .quantized.qconfig import QConfig, custom_mlu_qconfig, default_mlu_qconfig

_QUANT_TYPES = (nn.Linear, nn.Conv3d, nn.Conv2d, nn.Conv1d, "Conv2d")


def compose_qconfig(weight_observer, activation_observer):
    return QConfig(weight=weight_observer, activation=activation_observer)


def swap_module(mod, gen_quant, mapping):
    if type(mod) in mapping:
        return mapping[type(mod)].from_float(mod, gen_quant)
    if mod._get_name() in mapping:
        return mapping[mod._get_name()].from_float(mod, gen_quant)
    return mod


def convert(module, gen_quant, mapping=None, inplace=False):
    for name, child in list(module.named_children()):
        convert(child, gen_quant, mapping, inplace=True)
        module._modules[name] = swap_module(child, gen_quant, mapping)


def _observer_forward_hook(self, input, output):
    return self.observer(output)


def add_observer_(module):
    for child in module.children():
        if getattr(child, "qconfig", None) is not None:
            child.observer = child.qconfig.activation()
        else:
            add_observer_(child)
    if getattr(module, "qconfig", None) is not None and len(module._modules) == 0:
        module.add_module("observer", module.qconfig.activation())
        module.register_forward_hook(_observer_forward_hook)


def _propagate(module, qconfig_tuple, mixed_layer, white_list, parent_qconfig, prefix):
    spec = qconfig_tuple[1]
    if mixed_layer is not None:
        for names, dtype in mixed_layer.items():
            if prefix in [n.strip(" ") for n in names.split(",")] and dtype in {"float16", "int8", "int16"}:
                spec = {t: custom_mlu_qconfig(dtype, qconfig_tuple[0]) for t in _QUANT_TYPES}
    qc = spec.get(type(module), parent_qconfig)
    qc = spec.get(prefix, qc)
    qc = spec.get(module._get_name(), qc)
    qc = getattr(module, "qconfig", qc)
    if type(module) in white_list or module._get_name() in white_list:
        module.qconfig = qc
    for name, child in module.named_children():
        _propagate(child, qconfig_tuple, mixed_layer, white_list, qc, prefix + "." + name if prefix else name)


def propagate_qconfig_(module, qconfig_tuple=None, mixed_layer=None):
    _propagate(module, qconfig_tuple or {}, mixed_layer, DEFAULT_QCONFIG_PROPAGATE_WHITE_LIST, None, "")


def quantize_dynamic_mlu(model, qconfig_spec=None, dtype=None, mapping=None, inplace=False, gen_quant=False,
                         mixed_layer=None):
    if mixed_layer is not None:
        if not isinstance(mixed_layer, dict):
            raise ValueError("type(mixed_layer) must be dict, now is ", type(mixed_layer))
        print("The layers : ", list(mixed_layer.keys()), " will be quantized by ",
              list(mixed_layer.values())[0].strip(" "))
    user_spec = qconfig_spec
    if qconfig_spec is None:
        per_type = {t: default_mlu_qconfig for t in _QUANT_TYPES}
    elif isinstance(qconfig_spec, dict):
        if gen_quant:
            if dtype not in {"int8", "int16"}:
                raise ValueError("Unknow dtype for quantization")
            w_obs = mlu_weight_observer(dtype)
            if qconfig_spec.get("per_channel", False):
                w_obs = mlu_weight_per_channel_observer(dtype, qconfig_spec)
            a_obs = mlu_activation_observer_dict[qconfig_spec.get("method", "minmax")](dtype, qconfig_spec)
            per_type = {t: compose_qconfig(w_obs, a_obs) for t in _QUANT_TYPES}
            per_type[nn.Conv3d] = compose_qconfig(mlu_weight_observer(dtype), a_obs)  # 3-d: per-tensor weights only
        else:
            per_type = {t: custom_mlu_qconfig(dtype, qconfig_spec) for t in _QUANT_TYPES}
    else:
        raise ValueError("Unknown qconfig_spec")
    if mapping is None:
        mapping = DEFAULT_MLU_MODULE_MAPPING
    if not inplace:
        try:
            model = copy.deepcopy(model)
        except Exception:
            print('Warning: Failed to deepcopy model, "inplace" is set to True by default.')
    model.eval()
    propagate_qconfig_(model, [user_spec, per_type], mixed_layer)
    if gen_quant is True:
        add_observer_(model)
    if gen_quant:
        mapping[nn.Conv2d].is_first_layer = True  # a new calibration run starts with a new first layer
    convert(model, gen_quant, mapping, inplace=True)
    return model
