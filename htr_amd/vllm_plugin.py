"""vLLM quantization plugin for HTR-W1 checkpoints on MI355X (quant_method "htr", tensor parallel size 1).

Mirror of the in-scope part of the reference plugin (htr/vllm_plugin.py:1-150 of the reference): same class and parameter
names, same loader and selection rules, and `apply` ends in `ops.linear`, which here is the gfx950 library.  The
overlays for a private runtime image (htr/vllm_plugin.py:153-405) are not part of this build.

vLLM is imported when the module is imported, as in the reference.  Where it is not installed (this repository's test
environment), minimal stand-ins for the four vLLM names are used so that the selection and loading logic can be
exercised; `register()` refuses to run without the real package.
"""
import collections
import itertools
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


def canon(name):
    """Checkpoint/module name -> key of the `modules` table: no ".weight" suffix, path from the last "layers." on."""
    _, marker, tail = name.removesuffix(".weight").rpartition("layers.")
    return marker + tail


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

    def _width(self, prefix):
        """Bit width of the module at `prefix`, or None if the checkpoint does not quantize it.  A module that the
        model fuses from several checkpoint modules (packed_modules_mapping: qkv_proj <- q_proj, k_proj, v_proj) is
        looked up part by part: all parts quantized at one width, or none."""
        scope, dot, leaf = canon(prefix).rpartition(".")
        parts = (getattr(self, "packed_modules_mapping", None) or {}).get(leaf, [leaf])
        found = {part: self.modules.get(scope + dot + part) for part in parts}
        widths = set(found.values())
        if widths == {None}:
            return None
        if len(widths) > 1:
            raise ValueError(f"HTR: fused module {prefix} has mixed quantization {found}")
        return widths.pop()

    def get_quant_method(self, layer, prefix):
        if isinstance(layer, ParallelLMHead):
            # only an output head named lm_head that the checkpoint lists; other embeddings stay unquantized
            K = self.modules.get("lm_head") if prefix.split(".")[-1] == "lm_head" else None
            return None if K is None else HTRLinearMethod(K)
        if not isinstance(layer, LinearBase):
            return None
        in_skipped_tower = any(tag in prefix for tag in SKIP)
        K = None if in_skipped_tower else self._width(prefix)
        return UnquantizedLinearMethod() if K is None else HTRLinearMethod(K)


class _FusedRows:
    """Output-row layout of a module stacked from several parts (q | k | v, gate | up): which rows a checkpoint shard
    covers.  A shard is named by part index, by "q" / "k" / "v", by a run of consecutive part indices, or not at all
    (the whole module)."""
    NAMED = {"q": 0, "k": 1, "v": 2}

    def __init__(self, sizes):
        self.edges = list(itertools.accumulate(sizes, initial=0))      # part i covers rows edges[i] .. edges[i + 1]

    def rows(self, shard_id):
        last = len(self.edges) - 2
        if shard_id is None:
            lo, hi = 0, last
        elif isinstance(shard_id, (tuple, list)):
            lo, hi = shard_id[0], shard_id[-1]
            assert list(shard_id) == list(range(lo, hi + 1)), f"shard {shard_id} is not a run of consecutive parts"
        else:
            lo = hi = self.NAMED[shard_id] if isinstance(shard_id, str) else int(shard_id)
        assert 0 <= lo <= hi <= last, (shard_id, last)
        return self.edges[lo], self.edges[hi + 1]

    def span(self, shard_id, unit):
        """(first, count) of the shard in entries of `unit` output rows each."""
        r0, r1 = self.rows(shard_id)
        assert r0 % unit == 0 and r1 % unit == 0, (r0, r1, unit)
        return r0 // unit, (r1 - r0) // unit


def _shard_range(sizes, shard_id, unit):
    return _FusedRows(sizes).span(shard_id, unit)


class _RowPlacer:
    """weight_loader of a tensor indexed by output rows: a shard lands at its row offset, in the tensor's own unit."""

    def __init__(self, layout, unit):
        self.layout, self.unit = layout, unit

    def __call__(self, param, loaded, shard_id=None):
        if shard_id is None:
            shard_id = getattr(loaded, "shard_id", None)               # stacked-parameter mappers attach it to the tensor
        first, count = self.layout.span(shard_id, self.unit)
        dest = param.data.narrow(0, first, count)
        assert dest.shape == loaded.shape, (tuple(param.shape), tuple(loaded.shape), shard_id)
        dest.copy_(loaded)


class _SharedSigns:
    """weight_loader of the input sign vector: every part of a fused module brings the same one (docs/FORMAT.md:31-32);
    the first is kept, the others are compared with it."""

    def __init__(self):
        self.filled = False

    def __call__(self, param, loaded, shard_id=None):
        assert loaded.shape == param.shape
        if self.filled and not torch.equal(param.data.cpu(), loaded.cpu()):
            raise ValueError("HTR: fused shards do not share the input sign vector")
        if not self.filled:
            param.data.copy_(loaded)
            self.filled = True


# tensors indexed by output rows: name -> (dtype, output rows per entry of dim 0, trailing dims for n inputs at width K)
_ROW_TENSORS = {
    "htr_qweight": (torch.int32, 16, lambda n, K: (n // 16, 8 * K)),
    "htr_scales": (torch.float16, 1, lambda n, K: ()),
    "htr_sv": (torch.uint8, 8, lambda n, K: ()),
}


class HTRLinearMethod(LinearMethodBase):
    """Creates htr_qweight / htr_scales / htr_su / htr_sv on a linear layer and runs it through ops.linear."""

    def __init__(self, K):
        self.K = K

    def create_weights(self, layer, input_size_per_partition, output_partition_sizes, input_size, output_size,
                       params_dtype, **extra_weight_attrs):
        n, sizes = input_size_per_partition, list(output_partition_sizes)
        assert n == input_size, "HTR: tensor parallelism is not supported"
        assert n % 128 == 0 and all(s % 128 == 0 for s in sizes), (n, sizes)
        layout = _FusedRows(sizes)
        m = layout.edges[-1]

        def attach(name, tensor, loader):
            p = Parameter(tensor, requires_grad=False)
            layer.register_parameter(name, p)
            set_weight_attrs(p, {"weight_loader": loader})

        for name, (dtype, unit, trailing) in _ROW_TENSORS.items():
            attach(name, torch.empty((m // unit,) + trailing(n, self.K), dtype=dtype), _RowPlacer(layout, unit))
        attach("htr_su", torch.empty(n // 8, dtype=torch.uint8), _SharedSigns())
        layer.htr_K = self.K

    def process_weights_after_loading(self, layer):
        pass

    def apply(self, layer, x, bias=None):
        from . import ops
        if _COUNT_FILE is not None:
            _CENSUS.note(x.numel() // x.shape[-1], layer.htr_K)
        return ops.linear(x, layer.htr_qweight, layer.htr_scales, layer.htr_su, layer.htr_sv, bias)


# ---- dispatch census (HTR_COUNT_FILE=<path>): calls per batch bucket ("M1", "M2-8", "M>8") and per bit width ("K4"),
# written to <path>.<pid>.json every 512 calls through a temporary file and a rename
_COUNT_FILE = os.environ.get("HTR_COUNT_FILE") or None


class _Census:
    EVERY = 512

    def __init__(self):
        self.counts = collections.Counter()
        self.calls = 0

    def note(self, rows, K):
        self.counts["M1" if rows == 1 else "M2-8" if rows <= 8 else "M>8"] += 1
        self.counts[f"K{K}"] += 1
        self.calls += 1
        if self.calls % self.EVERY == 0:
            self.dump()

    def dump(self):
        final = f"{_COUNT_FILE}.{os.getpid()}.json"
        with open(final[:-5] + ".tmp", "w") as f:
            json.dump({"pid": os.getpid(), "t": time.time(), "counts": dict(self.counts)}, f)
        os.replace(final[:-5] + ".tmp", final)


_CENSUS = _Census()


def register():
    """vllm.general_plugins entry point: importing this module registered the "htr" method; make sure vLLM is there."""
    if not HAVE_VLLM:
        raise ImportError("htr_amd.vllm_plugin.register() needs vLLM; the quantization method cannot be registered without it")
    return HTRConfig
