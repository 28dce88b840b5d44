"""vLLM quantization plugin for HTR-W1 checkpoints on MI355X (quant_method "htr", tensor parallel size 1).

Mirror of the in-scope part of the reference plugin (htr/vllm_plugin.py:1-150 of the reference): same class and parameter
names, same loader and selection rules, and `apply` ends in `ops.linear`, which here is the gfx950 library.  The
overlays for a private runtime image (htr/vllm_plugin.py:153-405) are not part of this build.

vLLM is imported when the module is imported, as in the reference.  Where it is not installed (this repository's test
environment), minimal stand-ins for the four vLLM names are used so that the selection and loading logic can be
exercised; `register()` refuses to run without the real package.
"""
import collections
import json
import os
import time

import torch
from torch.nn import Parameter

try:  # pragma: no cover - exercised only where vLLM exists
    from vllm.model_executor.layers.linear import LinearBase, LinearMethodBase, UnquantizedLinearMethod
    from vllm.model_executor.layers.quantization import register_quantization_config
    from vllm.model_executor.layers.quantization.base_config import QuantizationConfig
    from vllm.model_executor.layers.vocab_parallel_embedding import ParallelLMHead
    from vllm.model_executor.utils import set_weight_attrs
    HAVE_VLLM = True
except ImportError:
    HAVE_VLLM = False

    class QuantizationConfig:                      # noqa: D401 - stand-in
        def __init__(self):
            self.packed_modules_mapping = {}

    class LinearBase(torch.nn.Module):
        pass

    class ParallelLMHead(torch.nn.Module):
        pass

    class LinearMethodBase:
        pass

    class UnquantizedLinearMethod(LinearMethodBase):
        pass

    def register_quantization_config(name):
        def deco(cls):
            return cls
        return deco

    def set_weight_attrs(weight, attrs):
        for k, v in attrs.items():
            setattr(weight, k, v)

# module-name fragments that are never quantized (vision / audio towers, multi-token-prediction heads)
SKIP = ("visual", "vision", "audio", "mtp")
_QKV_INDEX = {"q": 0, "k": 1, "v": 2}


def canon(name):
    """Checkpoint/module name -> key of the `modules` table: no ".weight" suffix, path from the last "layers." on."""
    if name.endswith(".weight"):
        name = name[:-len(".weight")]
    at = name.rfind("layers.")
    return name if at < 0 else name[at:]


@register_quantization_config("htr")
class HTRConfig(QuantizationConfig):
    """quantization_config {"quant_method": "htr", "wire": "HTR-W1", "modules": {prefix: {"K": k}}} (docs/FORMAT.md:34-36)."""

    def __init__(self, modules, wire="HTR-W1"):
        super().__init__()
        if wire != "HTR-W1":
            raise AssertionError(wire)
        self.modules = {canon(name): int(entry["K"]) for name, entry in modules.items()}

    def get_name(self):
        return "htr"

    def get_supported_act_dtypes(self):
        return [torch.bfloat16, torch.float16]

    @classmethod
    def get_min_capability(cls):
        return 0

    @staticmethod
    def get_config_filenames():
        return []

    @classmethod
    def from_config(cls, config):
        return cls(config.get("modules", {}), config.get("wire", "HTR-W1"))

    def get_quant_method(self, layer, prefix):
        parts = prefix.split(".")
        if isinstance(layer, ParallelLMHead):
            # only an output head named lm_head that the checkpoint lists; other embeddings stay unquantized
            K = self.modules.get("lm_head")
            return HTRLinearMethod(K) if K is not None and parts[-1] == "lm_head" else None
        if not isinstance(layer, LinearBase):
            return None
        if any(tag in parts or tag in prefix for tag in SKIP):
            return UnquantizedLinearMethod()
        key = canon(prefix)
        parent, _, leaf = key.rpartition(".")
        packed = getattr(self, "packed_modules_mapping", None) or {}
        members = packed.get(leaf, [leaf])
        widths = [self.modules.get(f"{parent}.{name}" if parent else name) for name in members]
        if all(k is None for k in widths):
            return UnquantizedLinearMethod()
        if None in widths or len(set(widths)) != 1:
            raise ValueError(f"HTR: fused module {prefix} has mixed quantization {dict(zip(members, widths))}")
        return HTRLinearMethod(widths[0])


def _shard_range(sizes, shard_id, unit):
    """(first, count) in `unit`-row units of the output rows that `shard_id` covers in a fused module."""
    if shard_id is None:
        picked = list(range(len(sizes)))
    elif isinstance(shard_id, str):
        picked = [_QKV_INDEX[shard_id]]
    elif isinstance(shard_id, (tuple, list)):
        picked = list(shard_id)
    else:
        picked = [int(shard_id)]
    if picked != list(range(picked[0], picked[-1] + 1)):
        raise AssertionError(picked)
    first = sum(sizes[:picked[0]])
    count = sum(sizes[i] for i in picked)
    if first % unit or count % unit:
        raise AssertionError((first, count, unit))
    return first // unit, count // unit


class HTRLinearMethod(LinearMethodBase):
    """Creates htr_qweight / htr_scales / htr_su / htr_sv on a linear layer and runs it through ops.linear."""

    def __init__(self, K):
        self.K = K

    def create_weights(self, layer, input_size_per_partition, output_partition_sizes, input_size, output_size,
                       params_dtype, **extra_weight_attrs):
        n, sizes = input_size_per_partition, list(output_partition_sizes)
        m = sum(sizes)
        assert input_size_per_partition == input_size, "HTR: tensor parallelism is not supported"
        assert n % 128 == 0 and all(s % 128 == 0 for s in sizes), (n, sizes)
        K = self.K
        tensors = {
            "htr_qweight": torch.empty(m // 16, n // 16, 8 * K, dtype=torch.int32),
            "htr_scales": torch.empty(m, dtype=torch.float16),
            "htr_su": torch.empty(n // 8, dtype=torch.uint8),
            "htr_sv": torch.empty(m // 8, dtype=torch.uint8),
        }

        def row_loader(unit):
            # qweight rows are 16 output rows, scales 1, sv 8: a fused shard lands at its row offset in those units
            def load(param, loaded, shard_id=None):
                if shard_id is None:
                    shard_id = getattr(loaded, "shard_id", None)      # stacked-parameter mappers attach it to the tensor
                first, count = _shard_range(sizes, shard_id, unit)
                assert tuple(loaded.shape) == (count,) + tuple(param.shape[1:]), (param.shape, loaded.shape, shard_id)
                param.data[first:first + count].copy_(loaded)
            return load

        def su_loader(param, loaded, shard_id=None):
            # the parts of a fused module must share the input sign vector (docs/FORMAT.md:31-32)
            assert loaded.shape == param.shape
            if getattr(param, "_htr_loaded", False):
                if not torch.equal(param.data.cpu(), loaded.cpu()):
                    raise ValueError("HTR: fused shards do not share the input sign vector")
                return
            param.data.copy_(loaded)
            param._htr_loaded = True

        loaders = {"htr_qweight": row_loader(16), "htr_scales": row_loader(1), "htr_sv": row_loader(8), "htr_su": su_loader}
        for name, value in tensors.items():
            p = Parameter(value, requires_grad=False)
            layer.register_parameter(name, p)
            set_weight_attrs(p, {"weight_loader": loaders[name]})
        layer.htr_K = K

    def process_weights_after_loading(self, layer):
        pass

    def apply(self, layer, x, bias=None):
        from . import ops
        if _COUNT_FILE is not None:
            _census(x, layer.htr_K)
        return ops.linear(x, layer.htr_qweight, layer.htr_scales, layer.htr_su, layer.htr_sv, bias)


# ---- dispatch census (HTR_COUNT_FILE): calls per batch bucket and per K, dumped atomically every 512 calls
_COUNT_FILE = os.environ.get("HTR_COUNT_FILE") or None
_COUNTS = collections.Counter()
_BUCKETS = ("M1", "M2-8", "M>8")


def _census(x, K):
    M = x.numel() // x.shape[-1]
    _COUNTS[_BUCKETS[0] if M == 1 else (_BUCKETS[1] if M <= 8 else _BUCKETS[2])] += 1
    _COUNTS["K%d" % K] += 1
    if sum(_COUNTS[b] for b in _BUCKETS) % 512 == 0:
        _dump_counts()


def _dump_counts():
    tmp = f"{_COUNT_FILE}.{os.getpid()}.tmp"
    with open(tmp, "w") as f:
        json.dump(dict(pid=os.getpid(), t=time.time(), counts=dict(_COUNTS)), f)
    os.replace(tmp, f"{_COUNT_FILE}.{os.getpid()}.json")


def register():
    """vllm.general_plugins entry point: importing this module registered the "htr" method; make sure vLLM is there."""
    if not HAVE_VLLM:
        raise ImportError("htr_amd.vllm_plugin.register() needs vLLM; the quantization method cannot be registered without it")
    return HTRConfig
