"""Ternary (Mode C / D) weights of a Boilerplate-format checkpoint directory as operands of the kernels.

What is read (layout: ``docs/architecture/format.md:87-134``; written by ``boilerplate/format/export.py:228-233``;
the reference reads it in ``boilerplate/engine/weights.py:93-159`` and builds its linears from it in
``boilerplate/engine/standard.py:36-42``):

* ``manifest.json``: ``{"format": "boilerplate", "version": 1, "tensors": {base: entry}}``; a ternary entry has
  ``mode`` "C" or "D", ``shape`` ``[N, K]``, ``packing`` ("tq1" / "tq2"), ``terms`` k, ``group``,
  ``scale_dtype``, ``act`` ("int8" / "bf16") and ``stored``: per stored tensor its dtype, shape, SHA-256 and,
  once sharded, the file that holds it;
* the stored tensors ``base.tq{i}.packed`` (uint8 ``[N, ceil(K / per_byte)]``) and ``base.tq{i}.scale``
  (fp16 / bf16 ``[N, ceil(K / group)]``), i = 0 .. k-1, in safetensors shards (``model.safetensors.index.json``
  maps names to files when present).

Every expert of an MoE layer is a weight of its own on disk; the grouped kernel wants one ``[E, N, Kp]`` stack per
term. ``stack`` fills such stacks expert by expert straight into device memory, so no second copy of a layer is
ever held on the host. Files are opened with ``safetensors.safe_open`` only: nothing in a checkpoint is executed.
Other modes (A: original dtype, B: entropy-coded) are not ternary and are refused here.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

from .ternary.ops import PackedTerm, TernaryLinear
from .ternary.pack import packed_cols

_SCALE_DTYPES = {"fp16": torch.float16, "float16": torch.float16, "bf16": torch.bfloat16, "bfloat16": torch.bfloat16}


def tensor_sha256(t: torch.Tensor) -> str:
    """SHA-256 of a tensor's bytes, as the exporter records it (boilerplate/format/export.py:70-71)."""
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


class TernaryCheckpoint:
    """Mode C / D weights of one checkpoint directory. ``verify=True`` checks every tensor read against the
    manifest's SHA-256 and raises ``ValueError`` on a mismatch."""

    def __init__(self, root: str | Path, verify: bool = False):
        self.root = Path(root)
        mpath = self.root / "manifest.json"
        if not mpath.exists():
            raise FileNotFoundError(f"{mpath}: not a Boilerplate-format checkpoint (no manifest.json)")
        self.manifest = json.loads(mpath.read_text())
        if self.manifest.get("format") != "boilerplate":
            raise ValueError(f"{mpath}: format {self.manifest.get('format')!r}, expected 'boilerplate'")
        if self.manifest.get("version") != 1:
            raise ValueError(f"{mpath}: manifest version {self.manifest.get('version')!r} is not supported (1 is)")
        self.verify = verify
        index = self.root / "model.safetensors.index.json"
        self._file_of: dict[str, str] = dict(json.loads(index.read_text())["weight_map"]) if index.exists() else {}
        self._handles: dict[str, object] = {}
        self._scanned = False

    # ------------------------------------------------------------------ manifest
    def bases(self) -> list[str]:
        """Base names of all ternary weights, in manifest order."""
        return [b for b, m in self.manifest["tensors"].items() if m.get("mode") in ("C", "D")]

    def entry(self, base: str) -> dict:
        try:
            m = self.manifest["tensors"][base]
        except KeyError:
            raise KeyError(f"{base!r} is not in the manifest of {self.root}") from None
        if m.get("mode") not in ("C", "D"):
            raise ValueError(f"{base!r} is stored in mode {m.get('mode')!r}; only ternary weights (C / D) are read here")
        for key in ("shape", "packing", "terms", "group"):
            if key not in m:
                raise ValueError(f"manifest entry of {base!r} has no {key!r}")
        return m

    # ------------------------------------------------------------------ tensors
    def _contained(self, fname: str) -> Path:
        """``root / fname`` for a file name that comes from the checkpoint itself (manifest, shard index), or
        ValueError: no absolute or drive paths, no backslashes, no ``.`` / ``..`` / empty components, and - after
        resolving symlinks - nothing outside the checkpoint directory (the rules of ``checkpoint_path``,
        boilerplate/checkpoint/paths.py:6-22)."""
        from pathlib import PurePosixPath, PureWindowsPath

        if (not isinstance(fname, str) or not fname or "\x00" in fname or "\\" in fname or PurePosixPath(fname).is_absolute()
                or PureWindowsPath(fname).drive or any(part in (".", "..", "") for part in fname.split("/"))):
            raise ValueError(f"unsafe checkpoint path: {fname!r}")
        root = self.root.resolve()
        path = (root / fname).resolve()
        if not path.is_relative_to(root):
            raise ValueError(f"checkpoint path escapes its directory: {fname!r}")
        return path

    def _open(self, fname: str):
        if fname not in self._handles:
            from safetensors import safe_open

            self._handles[fname] = safe_open(str(self._contained(fname)), framework="pt", device="cpu")
        return self._handles[fname]

    def _locate(self, name: str, stored: dict | None) -> str:
        if stored and "file" in stored:
            return stored["file"]
        if name in self._file_of:
            return self._file_of[name]
        if not self._scanned:  # no index: look into every shard once
            for p in sorted(self.root.glob("*.safetensors")):
                for n in self._open(p.name).keys():
                    self._file_of.setdefault(n, p.name)
            self._scanned = True
        if name not in self._file_of:
            raise KeyError(f"tensor {name!r} not in checkpoint {self.root}")
        return self._file_of[name]

    def tensor(self, name: str, stored: dict | None = None) -> torch.Tensor:
        """One stored tensor on the host; checked against ``stored`` (its manifest record) when given."""
        t = self._open(self._locate(name, stored)).get_tensor(name)
        if stored:
            if "shape" in stored and list(t.shape) != list(stored["shape"]):
                raise ValueError(f"{name}: shape {list(t.shape)} on disk, {stored['shape']} in the manifest")
            if self.verify and "sha256" in stored and tensor_sha256(t) != stored["sha256"]:
                raise ValueError(f"{name}: SHA-256 differs from the manifest")
        return t

    def terms(self, base: str) -> tuple[list[PackedTerm], dict]:
        """The k stacked terms of one weight (host tensors) and its manifest entry, shapes checked."""
        m = self.entry(base)
        N, K = m["shape"]
        Kp, G = packed_cols(m["packing"], K), -(-K // m["group"])
        want_scale = _SCALE_DTYPES.get(m.get("scale_dtype", "fp16"))
        out = []
        for i in range(m["terms"]):
            pn, sn = f"{base}.tq{i}.packed", f"{base}.tq{i}.scale"
            p = self.tensor(pn, m.get("stored", {}).get(pn))
            s = self.tensor(sn, m.get("stored", {}).get(sn))
            if p.dtype != torch.uint8 or tuple(p.shape) != (N, Kp):
                raise ValueError(f"{pn}: {p.dtype} {tuple(p.shape)}, expected uint8 {(N, Kp)} for {m['packing']} with K = {K}")
            if s.dtype not in (torch.float16, torch.bfloat16) or tuple(s.shape) != (N, G):
                raise ValueError(f"{sn}: {s.dtype} {tuple(s.shape)}, expected fp16 / bf16 {(N, G)} for group {m['group']}")
            if want_scale is not None and s.dtype != want_scale:
                raise ValueError(f"{sn}: stored as {s.dtype}, the manifest says {m['scale_dtype']}")
            out.append(PackedTerm(p, s))
        return out, m

    # ------------------------------------------------------------------ operands
    def linear(self, base: str, backend: str = "auto") -> TernaryLinear:
        """One weight as the reference builds it (boilerplate/engine/standard.py:37-41)."""
        terms, m = self.terms(base)
        return TernaryLinear(terms, m["shape"][1], m["packing"], m["group"], m.get("act", "int8"), backend=backend)

    def stack(self, bases: list[str], device) -> tuple[list[tuple[torch.Tensor, torch.Tensor]], dict]:
        """Weights of equal shape and coding as stacks ``(packed [E, N, Kp], scale [E, N, G])`` per term on
        ``device``, in the order of ``bases``; returns them with ``{"N", "K", "fmt", "group", "act", "terms"}``."""
        if not bases:
            raise ValueError("no weights to stack")
        first = self.entry(bases[0])
        key = lambda m: (tuple(m["shape"]), m["packing"], m["terms"], m["group"], m.get("scale_dtype", "fp16"), m.get("act", "int8"))  # noqa: E731
        N, K = first["shape"]
        Kp, G = packed_cols(first["packing"], K), -(-K // first["group"])
        sdt = _SCALE_DTYPES.get(first.get("scale_dtype", "fp16"), torch.float16)
        E = len(bases)
        out = [(torch.empty(E, N, Kp, dtype=torch.uint8, device=device), torch.empty(E, N, G, dtype=sdt, device=device))
               for _ in range(first["terms"])]
        for e, base in enumerate(bases):
            m = self.entry(base)
            if key(m) != key(first):
                raise ValueError(f"{base!r} ({key(m)}) does not match {bases[0]!r} ({key(first)}): cannot be stacked")
            terms, _ = self.terms(base)
            for (P, S), t in zip(out, terms):
                P[e].copy_(t.packed)
                S[e].copy_(t.scale)
        meta = {"N": N, "K": K, "fmt": first["packing"], "group": first["group"], "act": first.get("act", "int8"),
                "terms": first["terms"]}
        return out, meta

    def moe(self, expert_prefix: str, n_experts: int, top_k: int, device, names: tuple[str, str, str] = ("w1", "w3", "w2"),
            renorm: bool = False):
        """The routed experts ``expert_prefix.format(e) + "." + name`` as a ``TernaryMoE``; ``names`` = (gate, up,
        down): ``w1`` / ``w3`` / ``w2`` in the V4 engine's checkpoints (boilerplate/engine/model.py:373-375),
        ``gate_proj`` / ``up_proj`` / ``down_proj`` in the Llama / OLMoE ones (boilerplate/engine/standard.py:130-133)."""
        from .moe import TernaryMoE

        stacks, metas = [], []
        for name in names:
            st, meta = self.stack([f"{expert_prefix.format(e)}.{name}" for e in range(n_experts)], device)
            stacks.append(st)
            metas.append(meta)
        g, u, d = metas
        if (g["fmt"], g["group"], g["act"], g["terms"]) != (d["fmt"], d["group"], d["act"], d["terms"]) or \
                (g["fmt"], g["group"], g["act"], g["terms"], g["N"], g["K"]) != (u["fmt"], u["group"], u["act"], u["terms"], u["N"], u["K"]):
            raise ValueError("gate / up / down of the layer are coded differently; the grouped layer needs one coding")
        if (d["N"], d["K"]) != (g["K"], g["N"]):
            raise ValueError(f"down is {d['N']} x {d['K']}, expected {g['K']} x {g['N']}")
        return TernaryMoE(stacks[0], stacks[1], stacks[2], hidden=g["K"], inter=g["N"], top_k=top_k, fmt=g["fmt"],
                          group=g["group"], act=g["act"], renorm=renorm)
