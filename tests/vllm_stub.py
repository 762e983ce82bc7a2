"""A minimal stand-in for the parts of vLLM the plugin file imports, shaped after the interfaces in
the reference's tree (third_party/vllm-bitblas/vllm/model_executor/layers/linear.py:92-124,
.../quantization/base_config.py:58-135, vllm/model_executor/parameter.py): abstract bases with the
same abstract methods, parameter classes that keep their keyword arguments.  vLLM itself is not
installed where these tests run."""
import logging
import sys
import types
from abc import ABC, abstractmethod

import torch


class QuantizeMethodBase(ABC):
    @abstractmethod
    def create_weights(self, layer, *weight_args, **extra_weight_attrs):
        raise NotImplementedError

    @abstractmethod
    def apply(self, layer, *args, **kwargs):
        raise NotImplementedError

    def process_weights_after_loading(self, layer):
        return


class LinearMethodBase(QuantizeMethodBase):
    @abstractmethod
    def create_weights(self, layer, input_size_per_partition, output_partition_sizes, input_size, output_size,
                       params_dtype, **extra_weight_attrs):
        raise NotImplementedError

    @abstractmethod
    def apply(self, layer, x, bias=None):
        raise NotImplementedError


class LinearBase(torch.nn.Module):
    pass


class QuantizationConfig(ABC):
    @abstractmethod
    def get_name(self):
        raise NotImplementedError

    @abstractmethod
    def get_supported_act_dtypes(self):
        raise NotImplementedError

    @classmethod
    @abstractmethod
    def get_min_capability(cls):
        raise NotImplementedError

    @staticmethod
    @abstractmethod
    def get_config_filenames():
        raise NotImplementedError

    @classmethod
    @abstractmethod
    def from_config(cls, config):
        raise NotImplementedError

    @classmethod
    def override_quantization_method(cls, hf_quant_cfg, user_quant):
        return None

    @staticmethod
    def get_from_keys(config, keys):
        for key in keys:
            if key in config:
                return config[key]
        raise ValueError(f"Cannot find any of {keys} in the model's quantization config.")

    @abstractmethod
    def get_quant_method(self, layer, prefix):
        raise NotImplementedError


class _Param(torch.nn.Parameter):
    def __new__(cls, data, **kwargs):
        return super().__new__(cls, data=data, requires_grad=False)

    def __init__(self, data, **kwargs):
        self.attrs = kwargs


class PackedvLLMParameter(_Param):
    pass


class RowvLLMParameter(_Param):
    pass


class GroupQuantScaleParameter(_Param):
    pass


def install():
    """Register the stand-in modules under the names the plugin imports."""
    def module(name, **members):
        mod = types.ModuleType(name)
        mod.__dict__.update(members)
        sys.modules[name] = mod
        return mod

    module("vllm")
    module("vllm.logger", init_logger=logging.getLogger)
    module("vllm.model_executor")
    module("vllm.model_executor.layers")
    module("vllm.model_executor.layers.linear", LinearBase=LinearBase, LinearMethodBase=LinearMethodBase)
    module("vllm.model_executor.layers.quantization")
    module("vllm.model_executor.layers.quantization.base_config", QuantizationConfig=QuantizationConfig)
    module("vllm.model_executor.parameter", PackedvLLMParameter=PackedvLLMParameter,
           RowvLLMParameter=RowvLLMParameter, GroupQuantScaleParameter=GroupQuantScaleParameter)
