"""vLLM quantization plugin: ``--quantization qfactory`` served by this library's HIP kernels.

Install by copying this file to ``vllm/model_executor/layers/quantization/qfactory.py`` and adding
``"qfactory": QFactoryConfig`` to that package's method registry and ``"QFactoryLinearMethod"`` to
``WEIGHT_LOADER_V2_SUPPORTED`` in ``vllm/model_executor/layers/linear.py`` -- the same three edits as
the reference's patch (third_party/vllm-qfactory.patch:18-24, 39-44, 47-214).  Class names, method
names and signatures are those of the reference's file.

Differences from the reference's hook, all inside method bodies:

* ``process_weights_after_loading`` converts the loaded GPTQ tensors (qweight / qzeros / scales)
  into the packed layout and builds a working layer; the reference allocates an empty layer and
  never loads weights (vllm-qfactory.patch:188-203).
* the layer dispatches on the actual number of rows of ``x`` (prefill and decode share a layer).
* no on-device tiling search at load time (the analytic default, or ``$QFACTORY_CONFIG``).
* ``get_min_capability`` returns 0: the number is a CUDA SM version and means nothing on ROCm.
"""
from typing import Any, Dict, List, Optional

import torch

from vllm.logger import init_logger
from vllm.model_executor.layers.linear import LinearBase, LinearMethodBase
from vllm.model_executor.layers.quantization.base_config import QuantizationConfig
from vllm.model_executor.parameter import GroupQuantScaleParameter, PackedvLLMParameter, RowvLLMParameter

from qfactory import QLinear
from qfactory.integrations.gptq_format import gptq_to_qlinear_inputs

logger = init_logger(__name__)


class QFactoryConfig(QuantizationConfig):
    """Config class for QFactory (vllm-qfactory.patch:60-110)."""

    def __init__(self, weight_bits: int, group_size: int):
        self.weight_bits = weight_bits
        self.pack_factor = 32 // weight_bits
        self.group_size = group_size

    def __repr__(self) -> str:
        return f"QFactoryConfig(weight_bits={self.weight_bits}, group_size={self.group_size})"

    @classmethod
    def from_config(cls, config: Dict[str, Any]) -> "QFactoryConfig":
        weight_bits = cls.get_from_keys(config, ["bits"])
        group_size = cls.get_from_keys(config, ["group_size"])
        return cls(weight_bits, group_size)

    @classmethod
    def override_quantization_method(cls, hf_quant_cfg, user_quant) -> Optional[str]:
        if user_quant == "qfactory":
            logger.warning("Using qfactory kernel.")
            return user_quant
        return None

    @classmethod
    def get_min_capability(cls) -> int:
        return 0

    def get_supported_act_dtypes(self) -> List[torch.dtype]:
        return [torch.float16]

    def get_quant_method(self, layer: torch.nn.Module, prefix: str) -> Optional["QFactoryLinearMethod"]:
        if isinstance(layer, LinearBase):
            return QFactoryLinearMethod(self, prefix)
        return None

    def get_name(self) -> str:
        return "qfactory"

    @staticmethod
    def get_config_filenames() -> List[str]:
        raise NotImplementedError


class QFactoryLinearMethod(LinearMethodBase):
    """Linear method for QFactory (vllm-qfactory.patch:113-214)."""

    def __init__(self, quant_config: QFactoryConfig, prefix: str):
        self.quant_config = quant_config
        self.prefix = prefix

    def create_weights(self, layer: torch.nn.Module, input_size_per_partition: int,
                       output_partition_sizes: List[int], input_size: int, output_size: int,
                       params_dtype: torch.dtype, **extra_weight_attrs):
        cfg = self.quant_config
        output_size_per_partition = sum(output_partition_sizes)
        weight_loader = extra_weight_attrs.get("weight_loader")
        groups = input_size_per_partition // cfg.group_size

        qweight = PackedvLLMParameter(
            data=torch.empty(input_size_per_partition // cfg.pack_factor, output_size_per_partition, dtype=torch.int32),
            input_dim=0, output_dim=1, packed_dim=0, packed_factor=cfg.pack_factor, weight_loader=weight_loader)
        # starts as the trivial map k // group_size: a checkpoint without a g_idx tensor (older exports with
        # desc_act=False) then means "no reordering" instead of leaving uninitialised memory for the check below
        g_idx = RowvLLMParameter(
            data=(torch.arange(input_size_per_partition, dtype=torch.int32) // cfg.group_size),
            input_dim=0, weight_loader=weight_loader)
        scales = GroupQuantScaleParameter(
            data=torch.empty(groups, output_size_per_partition, dtype=params_dtype),
            input_dim=0, output_dim=1, weight_loader=weight_loader)
        qzeros = PackedvLLMParameter(
            data=torch.empty(groups, output_size_per_partition // cfg.pack_factor, dtype=torch.int32),
            input_dim=0, output_dim=1, packed_dim=1, packed_factor=cfg.pack_factor, weight_loader=weight_loader)

        layer.register_parameter("qweight", qweight)
        layer.register_parameter("g_idx", g_idx)
        layer.register_parameter("scales", scales)
        layer.register_parameter("qzeros", qzeros)

    def process_weights_after_loading(self, layer: torch.nn.Module):
        cfg = self.quant_config
        input_size = layer.qweight.shape[0] * cfg.pack_factor
        output_size = layer.qweight.shape[1]
        # the loaded g_idx decides: only the trivial k // group_size is computed correctly here, anything else
        # (an activation-reordered, desc_act checkpoint) raises NotImplementedError instead of loading
        weight, scale, zero = gptq_to_qlinear_inputs(layer.qweight.data, layer.qzeros.data, layer.scales.data,
                                                     cfg.weight_bits, cfg.group_size, g_idx=layer.g_idx.data)
        layer.qlinear = QLinear.init(
            1, input_size, output_size, cfg.weight_bits, weight, cfg.group_size, scale, zero,
            compile_flags={"enable_transform": False, "enable_schedule": False, "enable_lower": False})
        layer.register_parameter("qweight", None)
        layer.register_parameter("qzeros", None)
        layer.register_parameter("scales", None)
        layer.register_parameter("g_idx", None)

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Apply the weights in layer to the input tensor.
        Expects create_weights to have been called before on the layer."""
        lead = x.shape[:-1]
        out = layer.qlinear(x.reshape(-1, x.shape[-1]).contiguous())
        if bias is not None:
            out.add_(bias)
        return out.reshape(*lead, out.shape[-1])
