"""Reader for HTR-W1 checkpoints: safetensors shards with `<prefix>.htr_{qweight,scales,su,sv}` per quantized linear and
the table of bit widths in config.json.

Layout written by the reference's converters (docs/FORMAT.md:25-36; htr/quantize.py:252-289 writes
`quantization_config = {"quant_method": "htr", "wire": "HTR-W1", "generator": "rdna24", "L": 16, "tile": 16,
"rht_block": 128, "modules": {prefix: {"K": k}}}`; htr/encode_q38.py:205-209 nests the same table as
`quantization_config["htr_overlay"]` under another quant method).  Nothing here executes anything from the files:
safetensors and JSON only.
"""
import json
import os

import torch

from . import wire

SUFFIXES = ("htr_qweight", "htr_scales", "htr_su", "htr_sv")
_EXPECT = {"wire": wire.WIRE_NAME, "generator": "rdna24", "L": wire.L, "tile": wire.TILE, "rht_block": wire.RHT_BLOCK}


def read_quantization_config(config):
    """config: path of config.json, or its dict.  Returns {prefix: K}; raises ValueError for another wire or generator."""
    if not isinstance(config, dict):
        with open(config) as f:
            config = json.load(f)
    qc = config.get("quantization_config") or {}
    table = qc if qc.get("quant_method") == "htr" else qc.get("htr_overlay")
    if table is None:
        raise ValueError("config has no HTR quantization table (quant_method 'htr' or an 'htr_overlay' entry)")
    for key, want in _EXPECT.items():
        if key in table and table[key] != want:
            raise ValueError(f"unsupported HTR checkpoint: {key} = {table[key]!r}, this build reads {want!r}")
    mods = {name: int(entry["K"]) for name, entry in table.get("modules", {}).items()}
    for name, k in mods.items():
        if not 2 <= k <= 8:
            raise ValueError(f"{name}: K = {k} outside 2..8")
    return mods


class Checkpoint:
    """Lazy view of a checkpoint directory (or a single .safetensors file)."""

    def __init__(self, path):
        from safetensors import safe_open
        self._open = safe_open
        self.path = path
        if os.path.isdir(path):
            index = os.path.join(path, "model.safetensors.index.json")
            if os.path.exists(index):
                with open(index) as f:
                    wm = json.load(f)["weight_map"]
                self.weight_map = {k: os.path.join(path, v) for k, v in wm.items()}
            else:
                self.weight_map = {}
                for fn in sorted(os.listdir(path)):
                    if fn.endswith(".safetensors"):
                        with safe_open(os.path.join(path, fn), "pt") as fh:
                            for k in fh.keys():
                                self.weight_map[k] = os.path.join(path, fn)
            cfg = os.path.join(path, "config.json")
            self.modules = read_quantization_config(cfg) if os.path.exists(cfg) else None
        else:
            with safe_open(path, "pt") as fh:
                self.weight_map = {k: path for k in fh.keys()}
            self.modules = None

    def prefixes(self):
        """Prefixes that carry a complete HTR-W1 tensor set."""
        have = {}
        for key in self.weight_map:
            pre, _, suf = key.rpartition(".")
            if suf in SUFFIXES:
                have.setdefault(pre, set()).add(suf)
        return sorted(p for p, s in have.items() if s == set(SUFFIXES))

    def _tensor(self, key, device):
        if key not in self.weight_map:
            raise KeyError(key)
        with self._open(self.weight_map[key], "pt") as fh:
            return fh.get_tensor(key).to(device)

    def linear(self, prefix, device="cpu"):
        """(qweight, scales, su, sv) of one quantized linear, validated against the wire and the config's K."""
        t = tuple(self._tensor(f"{prefix}.{s}", device) for s in SUFFIXES)
        m, n, K = wire.check_shapes(*t)
        if self.modules is not None:
            want = self.modules.get(prefix)
            if want is not None and want != K:
                raise ValueError(f"{prefix}: tensors have K = {K}, config says {want}")
        return t

    def fused(self, prefixes, device="cpu"):
        """Several linears over the same input as one HTR-W1 tensor set (q/k/v, gate/up): qweight, scales and sv
        concatenate along the output dim; the parts must share su and K (docs/FORMAT.md:31-32)."""
        parts = [self.linear(p, device) for p in prefixes]
        ks = {wire.bits_of(p[0]) for p in parts}
        if len(ks) != 1:
            raise ValueError(f"fused parts {list(prefixes)} have different K {sorted(ks)}")
        su = parts[0][2]
        for p, name in zip(parts[1:], list(prefixes)[1:]):
            if not torch.equal(p[2], su):
                raise ValueError(f"fused part {name} does not share the input sign vector")
        return (torch.cat([p[0] for p in parts]).contiguous(), torch.cat([p[1] for p in parts]).contiguous(), su,
                torch.cat([p[3] for p in parts]).contiguous())


def save_linears(path, linears, metadata=None):
    """Write {prefix: (qweight, scales, su, sv)} as one safetensors file (the layout `Checkpoint` reads)."""
    from safetensors.torch import save_file
    flat = {}
    for prefix, t in linears.items():
        wire.check_shapes(*t)
        for suf, v in zip(SUFFIXES, t):
            flat[f"{prefix}.{suf}"] = v.detach().cpu().clone().contiguous()      # own storage: parts of a fused module share su
    save_file(flat, path, metadata={"format": "pt", **(metadata or {})})


def quantization_config(linears):
    """The `quantization_config` entry of config.json for {prefix: (qweight, scales, su, sv)}, as the reference's
    converter writes it (htr/quantize.py:282-283): wire, generator and geometry constants plus the bit width per module."""
    return {"quant_method": "htr", **_EXPECT,
            "modules": {prefix: {"K": wire.check_shapes(*t)[2]} for prefix, t in linears.items()}}


def save_checkpoint(directory, linears, config=None):
    """A checkpoint directory `Checkpoint` (and the plugin's HTRConfig.from_config) can read: model.safetensors with the
    packed tensors and config.json = `config` (a dict, e.g. the dense model's) with the HTR table put in."""
    os.makedirs(directory, exist_ok=True)
    save_linears(os.path.join(directory, "model.safetensors"), linears)
    cfg = dict(config or {})
    cfg["quantization_config"] = quantization_config(linears)
    with open(os.path.join(directory, "config.json"), "w") as f:
        json.dump(cfg, f, indent=2)
    return cfg
