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


# ------------------------------------------------------------------------------------------------ routed-expert chunks
# The reference's routed-expert encoder (htr/moe_encode.py:26-29, 216-225) writes, per layer L and per run of `chunk`
# consecutive experts starting at e0, one file <root>/L<L>/c<e0:03d>.pt = torch.save of
#   {"format": "HTR-W1-P2-PACKED-1", "L": L, "K": K,
#    "experts": [{"e": id, "n": calibration rows, "packed": {role: {"qweight", "scales", "su", "sv"}},
#                 "what_bf16_sha256": {role: hex}}, ...], "rows": [...], ...}
# with role in ("gate", "up", "down"), and <root>/PLAN.json with the run's arguments and the same format string.  The
# sha256 is over the BF16 bits of the encoder's reconstruction, which the encoder checked to equal wire.dequant of the
# packed tensors bit for bit (htr/moe_encode.py:63-75), so a reader can check a chunk without the encoder.
PACKED_FORMAT = "HTR-W1-P2-PACKED-1"
ROLES = ("gate", "up", "down")
FIELDS = ("qweight", "scales", "su", "sv")


def _chunk_name(e0):
    return f"c{e0:03d}.pt"


def write_packed_chunk(path, L, K, experts, extra=None):
    """Write one chunk file.  experts: iterable of {"e": id, "n": rows, "packed": {role: (qweight, scales, su, sv)}};
    the reconstruction hashes are computed here from wire.dequant.  For tests and for converters on this side: the
    reference's own encoder is the normal producer."""
    import hashlib
    out = []
    for ex in experts:
        packed, sha = {}, {}
        for role in ROLES:
            t = tuple(v.detach().cpu().contiguous() for v in ex["packed"][role])
            if wire.check_shapes(*t)[2] != K:
                raise ValueError(f"expert {ex['e']} {role}: tensors are not K = {K}")
            packed[role] = dict(zip(FIELDS, t))
            sha[role] = hashlib.sha256(wire.dequant(*t).bfloat16().contiguous().view(torch.int16).numpy().tobytes()).hexdigest()
        out.append({"e": int(ex["e"]), "n": int(ex.get("n", 0)), "packed": packed, "what_bf16_sha256": sha})
    z = {"format": PACKED_FORMAT, "L": int(L), "K": int(K), "experts": out, "rows": [], **(extra or {})}
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    torch.save(z, path)
    return z


def read_packed_chunk(path, device="cpu", verify=False):
    """One chunk file -> {"L", "K", "experts": {e: {"n", "gate", "up", "down", "what_bf16_sha256"}}} with every role an
    HTR-W1 tuple (qweight, scales, su, sv) on `device`.  The file is unpickled with torch's weights-only loader: tensors,
    numbers, strings, lists and dicts, nothing that runs code.  Shapes, K and the MLP structure are always checked; the
    encoder's reconstruction hashes (what_bf16_sha256) are NOT, unless asked for: verify=True recomputes all of them
    (decodes every matrix on the host with torch: about a second per real expert matrix), verify="first" only those of
    the chunk's first expert (a cheap guard against a chunk written with another codebook or bit order)."""
    z = torch.load(path, map_location="cpu", weights_only=True)
    if not isinstance(z, dict) or z.get("format") != PACKED_FORMAT:
        raise ValueError(f"{path}: not a {PACKED_FORMAT} chunk (format = {z.get('format') if isinstance(z, dict) else type(z).__name__!r})")
    K = int(z["K"])
    if not 2 <= K <= 8:
        raise ValueError(f"{path}: K = {K} outside 2..8")
    experts = {}
    for pos, ex in enumerate(z["experts"]):
        e = int(ex["e"])
        if e in experts:
            raise ValueError(f"{path}: expert {e} appears twice")
        rec = {"n": int(ex.get("n", 0)), "what_bf16_sha256": dict(ex.get("what_bf16_sha256") or {})}
        for role in ROLES:
            fields = ex["packed"][role]
            t = tuple(fields[f] for f in FIELDS)
            m, n, k = wire.check_shapes(*t)
            if k != K:
                raise ValueError(f"{path}: expert {e} {role} has K = {k}, the chunk says {K}")
            if verify is True or (verify == "first" and pos == 0):
                import hashlib
                got = hashlib.sha256(wire.dequant(*t).bfloat16().contiguous().view(torch.int16).numpy().tobytes()).hexdigest()
                want = rec["what_bf16_sha256"].get(role)
                if want != got:
                    raise ValueError(f"{path}: expert {e} {role}: decoded matrix does not match the encoder's reconstruction hash")
            rec[role] = tuple(v.to(device) for v in t)
        if rec["gate"][0].shape != rec["up"][0].shape or rec["down"][0].shape[0] * 16 != rec["gate"][2].numel() * 8:
            raise ValueError(f"{path}: expert {e}: gate/up/down shapes do not form an MLP")
        experts[e] = rec
    return {"L": int(z["L"]), "K": K, "experts": experts}


def fuse_gate_up(gate, up):
    """gate and up of one expert as the fused [2F, H] HTR-W1 tuple ops.moe_experts takes (gate rows first).  They
    share the input, so they must share su (the encoder draws one su per group: htr/moe_encode.py:199 shared_su)."""
    if not torch.equal(gate[2], up[2]):
        raise ValueError("gate and up do not share the input sign vector: they cannot run as one fused matrix")
    return (torch.cat([gate[0], up[0]]).contiguous(), torch.cat([gate[1], up[1]]).contiguous(), gate[2],
            torch.cat([gate[3], up[3]]).contiguous())


class PackedExperts:
    """A directory of routed-expert chunks: <root>/PLAN.json (optional) and <root>/L<L>/c<e0:03d>.pt."""

    def __init__(self, root):
        self.root = root
        self.plan = None
        pf = os.path.join(root, "PLAN.json")
        if os.path.exists(pf):
            with open(pf) as f:
                self.plan = json.load(f)
            if self.plan.get("format") != PACKED_FORMAT:
                raise ValueError(f"{pf}: format {self.plan.get('format')!r}, this build reads {PACKED_FORMAT!r}")

    def layers(self):
        out = []
        for d in os.listdir(self.root):
            if d.startswith("L") and d[1:].isdigit() and os.path.isdir(os.path.join(self.root, d)):
                out.append(int(d[1:]))
        return sorted(out)

    def chunks(self, L):
        """Paths of layer L's finished chunks in expert order (claims and temporary files of running encoders are skipped)."""
        d = os.path.join(self.root, f"L{L}")
        names = [fn for fn in os.listdir(d) if fn.startswith("c") and fn.endswith(".pt") and fn[1:-3].isdigit()]
        return [os.path.join(d, fn) for fn in sorted(names, key=lambda fn: int(fn[1:-3]))]

    def layer(self, L, device="cpu", verify=False):
        """(gate_up, down, K): lists indexed by expert id, ready for ops.moe_experts.  Raises if the layer's chunks leave
        a hole in the expert ids, disagree in K, or name another layer.  The reconstruction hashes in the chunks go
        unchecked by default; verify="first" checks the first expert of every chunk, verify=True all of them (see
        read_packed_chunk for the cost)."""
        recs, K = {}, None
        for p in self.chunks(L):
            z = read_packed_chunk(p, device, verify)
            if z["L"] != L:
                raise ValueError(f"{p}: chunk of layer {z['L']} under L{L}")
            if K is not None and z["K"] != K:
                raise ValueError(f"{p}: K = {z['K']}, earlier chunks of the layer have {K}")
            K = z["K"]
            for e, rec in z["experts"].items():
                if e in recs:
                    raise ValueError(f"{p}: expert {e} is in two chunks")
                recs[e] = rec
        if not recs:
            raise FileNotFoundError(f"no chunks for layer {L} under {self.root}")
        if sorted(recs) != list(range(len(recs))):
            raise ValueError(f"layer {L}: expert ids {sorted(recs)[:4]}.. are not 0..{len(recs) - 1} (chunks missing?)")
        gate_up = [fuse_gate_up(recs[e]["gate"], recs[e]["up"]) for e in range(len(recs))]
        down = [recs[e]["down"] for e in range(len(recs))]
        return gate_up, down, K
