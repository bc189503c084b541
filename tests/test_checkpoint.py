"""The Mode C / D checkpoint reader against directories written here in the reference's on-disk layout
(docs/architecture/format.md:87-134): manifest checks, shapes, SHA-256, stacking of per-expert weights; and against
tests/golden/export_tiny, two checkpoints written by the reference's own exporter (boilerplate/format/export.py:115-300,
run by tests/golden/make_export_fixture.py)."""

import json

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from _util import orc, synth_weights

from deepseekternarized_amd.checkpoint import TernaryCheckpoint, tensor_sha256

GROUP = 128


def _write(root, weights, shards=2, index=True, with_file=True):
    """weights: {base: (fmt, N, K, terms, packed list [N, Kp], scales list [N, G], act)}"""
    tensors, manifest = {}, {"format": "boilerplate", "version": 1, "tensors": {}}
    for base, (fmt, N, K, terms, packed, scales, act) in weights.items():
        stored = {}
        for i in range(terms):
            tensors[f"{base}.tq{i}.packed"] = torch.from_numpy(np.ascontiguousarray(packed[i]))
            tensors[f"{base}.tq{i}.scale"] = torch.from_numpy(np.ascontiguousarray(scales[i]))
            for n in (f"{base}.tq{i}.packed", f"{base}.tq{i}.scale"):
                t = tensors[n]
                stored[n] = {"dtype": str(t.dtype).replace("torch.", ""), "shape": list(t.shape), "sha256": tensor_sha256(t)}
        manifest["tensors"][base] = {"mode": "C", "shape": [N, K], "packing": fmt, "terms": terms, "group": GROUP,
                                     "scale_dtype": "fp16", "act": act, "gptq": False, "stored": stored}
    names = sorted(tensors)
    weight_map = {}
    for s in range(shards):
        part = {n: tensors[n] for n in names[s::shards]}
        fname = f"model-{s + 1:05d}-of-{shards:05d}.safetensors"
        save_file(part, str(root / fname))
        for n in part:
            weight_map[n] = fname
    if with_file:
        for m in manifest["tensors"].values():
            for n, rec in m["stored"].items():
                rec["file"] = weight_map[n]
    if index:
        (root / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    manifest["tensors"]["layers.0.attn.wq"] = {"mode": "A", "shape": [8, 8]}
    (root / "manifest.json").write_text(json.dumps(manifest))
    return tensors


def _experts(fmt, E, N, K, terms, seed, prefix="layers.0.ffn.experts", name="w1", act="int8"):
    packed, scales = synth_weights(seed, E, N, K, GROUP, fmt, terms=terms)
    return {f"{prefix}.{e}.{name}": (fmt, N, K, terms, [p[e] for p in packed], [s[e] for s in scales], act) for e in range(E)}, packed, scales


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("layout", ["index", "file", "scan"])
def test_terms_and_stack_match_what_was_written(tmp_path, fmt, layout):
    w, packed, scales = _experts(fmt, 3, 16, 1280, 2, seed=1)
    _write(tmp_path, w, index=layout == "index", with_file=layout == "file")
    ck = TernaryCheckpoint(tmp_path, verify=True)
    assert ck.bases() == list(w)
    terms, meta = ck.terms("layers.0.ffn.experts.1.w1")
    assert meta["packing"] == fmt and len(terms) == 2
    assert np.array_equal(terms[1].packed.numpy(), packed[1][1]) and np.array_equal(terms[1].scale.numpy(), scales[1][1])
    stacks, m = ck.stack(list(w), "cpu")
    assert m == {"N": 16, "K": 1280, "fmt": fmt, "group": GROUP, "act": "int8", "terms": 2}
    for i in range(2):
        assert stacks[i][0].shape == packed[i].shape and stacks[i][0].dtype == torch.uint8
        assert np.array_equal(stacks[i][0].numpy(), packed[i]) and np.array_equal(stacks[i][1].numpy(), scales[i])
    lin = ck.linear("layers.0.ffn.experts.2.w1")
    assert (lin.K, lin.fmt, lin.group, lin.act, lin.out_features) == (1280, fmt, GROUP, "int8", 16)


def test_refusals(tmp_path):
    w, _, _ = _experts("tq2", 2, 16, 1024, 1, seed=2)
    other, _, _ = _experts("tq1", 1, 16, 1024, 1, seed=3, prefix="layers.1.ffn.experts")
    tensors = _write(tmp_path, {**w, **other})
    ck = TernaryCheckpoint(tmp_path)
    with pytest.raises(ValueError, match="mode 'A'"):
        ck.entry("layers.0.attn.wq")
    with pytest.raises(KeyError):
        ck.entry("layers.9.nope")
    with pytest.raises(ValueError, match="cannot be stacked"):
        ck.stack(list(w) + list(other), "cpu")
    with pytest.raises(ValueError, match="no weights"):
        ck.stack([], "cpu")
    # a manifest that disagrees with the file
    man = json.loads((tmp_path / "manifest.json").read_text())
    base = "layers.0.ffn.experts.0.w1"
    man["tensors"][base]["shape"] = [16, 2048]
    (tmp_path / "manifest.json").write_text(json.dumps(man))
    with pytest.raises(ValueError, match="expected uint8"):
        TernaryCheckpoint(tmp_path).terms(base)
    man["tensors"][base]["shape"] = [16, 1024]
    man["tensors"][base]["stored"][base + ".tq0.packed"]["sha256"] = "0" * 64
    (tmp_path / "manifest.json").write_text(json.dumps(man))
    TernaryCheckpoint(tmp_path).terms(base)  # not checked unless asked
    with pytest.raises(ValueError, match="SHA-256"):
        TernaryCheckpoint(tmp_path, verify=True).terms(base)
    assert tensor_sha256(tensors[base + ".tq0.scale"]) == man["tensors"][base]["stored"][base + ".tq0.scale"]["sha256"]
    man["format"] = "gguf"
    (tmp_path / "manifest.json").write_text(json.dumps(man))
    with pytest.raises(ValueError, match="format"):
        TernaryCheckpoint(tmp_path)
    (tmp_path / "manifest.json").unlink()
    with pytest.raises(FileNotFoundError):
        TernaryCheckpoint(tmp_path)


@pytest.mark.gpu
def test_linear_and_moe_from_checkpoint_match_the_oracle(tmp_path):
    """A checkpoint with one MoE layer (4 experts, gate / up / down, two terms) read back and run on the GPU."""
    import deepseekternarized_amd as bp
    from _util import c_gemm

    H, I, E, k = 1024, 256, 4, 2
    ws, stacks = {}, {}
    for name, (N, K), seed in (("w1", (I, H), 5), ("w3", (I, H), 6), ("w2", (H, I), 7)):
        w, packed, scales = _experts("tq2", E, N, K, 2, seed=seed, name=name, act="bf16")
        ws.update(w)
        stacks[name] = (packed, scales)
    _write(tmp_path, ws, shards=3)
    ck = TernaryCheckpoint(tmp_path, verify=True)
    rng = np.random.default_rng(0)
    x = orc.bf16_round(rng.standard_normal((5, H)).astype(np.float32))
    # one linear
    lin = ck.linear("layers.0.ffn.experts.3.w1")
    got = lin(torch.from_numpy(x).cuda().to(torch.bfloat16), out_dtype=torch.float32).cpu().numpy()
    want = np.zeros((5, I), np.float32)
    for p, s in zip(*stacks["w1"]):
        c_gemm(x, None, p[3], s[3].astype(np.float32), H, GROUP, "tq2", out=want)
    assert np.linalg.norm(got - want) <= 1e-2 * np.linalg.norm(want)  # bf16 output rounding
    # the layer: same result as a TernaryMoE built from the stacks that were written
    moe = ck.moe("layers.0.ffn.experts.{}", E, k, "cuda")
    from deepseekternarized_amd.moe import TernaryMoE

    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    ref = TernaryMoE(*[[(dev(p), dev(s)) for p, s in zip(*stacks[n])] for n in ("w1", "w3", "w2")], hidden=H, inter=I, top_k=k,
                     fmt="tq2", group=GROUP, act="bf16")
    xd = dev(x).to(torch.bfloat16)
    logits = dev(rng.standard_normal((5, E)).astype(np.float32))
    a, b = moe(xd, logits), ref(xd, logits)
    assert torch.equal(a, b) and torch.isfinite(a).all()
    assert bp.ext() is not None


@pytest.mark.parametrize("bad", ["../outside.safetensors", "/etc/passwd", "sub/../../x.safetensors", "a\\b.safetensors", "./x.safetensors", ""])
@pytest.mark.parametrize("where", ["manifest", "index"])
def test_file_names_from_the_checkpoint_cannot_leave_its_directory(tmp_path, bad, where):
    """boilerplate/checkpoint/paths.py:6-22: names that come from manifest.json or the shard index are confined to the
    checkpoint directory (no absolute paths, `..`, backslashes, empty components, or symlinks that lead outside)."""
    root = tmp_path / "ck"
    root.mkdir()
    w, _, _ = _experts("tq2", 1, 16, 1280, 1, seed=3)
    _write(root, w, shards=1, index=True, with_file=True)
    base = next(iter(w))
    if where == "manifest":
        m = json.loads((root / "manifest.json").read_text())
        for rec in m["tensors"][base]["stored"].values():
            rec["file"] = bad
        (root / "manifest.json").write_text(json.dumps(m))
    else:
        m = json.loads((root / "manifest.json").read_text())
        for rec in m["tensors"][base]["stored"].values():
            rec.pop("file", None)
        (root / "manifest.json").write_text(json.dumps(m))
        idx = json.loads((root / "model.safetensors.index.json").read_text())
        idx["weight_map"] = {n: bad for n in idx["weight_map"]}
        (root / "model.safetensors.index.json").write_text(json.dumps(idx))
    ck = TernaryCheckpoint(root)
    with pytest.raises(ValueError, match="checkpoint path"):
        ck.terms(base)


def test_symlinked_shard_outside_the_directory_is_refused(tmp_path):
    root, outside = tmp_path / "ck", tmp_path / "elsewhere"
    root.mkdir()
    outside.mkdir()
    w, _, _ = _experts("tq2", 1, 16, 1280, 1, seed=4)
    _write(root, w, shards=1, index=True, with_file=True)
    shard = next(root.glob("*.safetensors"))
    moved = outside / shard.name
    shard.rename(moved)
    shard.symlink_to(moved)
    with pytest.raises(ValueError, match="escapes"):
        TernaryCheckpoint(root).terms(next(iter(w)))


# --------------------------------------------------------------------------- checkpoints written by the reference's exporter
from pathlib import Path  # noqa: E402

EXPORTS = Path(__file__).resolve().parent / "golden" / "export_tiny"
EXPERT_BASES = [f"layers.0.ffn.experts.{e}.{w}" for e in range(2) for w in ("w1", "w2", "w3")]


def _source():
    from safetensors import safe_open

    with safe_open(str(EXPORTS / "source" / "weights.safetensors"), framework="pt", device="cpu") as f:
        return {n: f.get_tensor(n) for n in f.keys()}


@pytest.mark.parametrize("name,mode,fmt,terms,group,sdt,act", [("mode_c_tq1", "C", "tq1", 2, 128, torch.float16, "int8"),
                                                                ("mode_d_tq2", "D", "tq2", 1, 64, torch.bfloat16, "bf16")])
def test_reads_what_the_reference_exporter_wrote(name, mode, fmt, terms, group, sdt, act):
    """Names, `terms`, `group`, `scale_dtype`, `act`, shapes and SHA-256 of every stored tensor as the reference's exporter
    recorded them (boilerplate/format/export.py:204-234); the dense weight no rule matched stays Mode A and is refused."""
    ck = TernaryCheckpoint(EXPORTS / name, verify=True)
    assert ck.bases() == sorted(EXPERT_BASES)
    src = _source()
    for base in EXPERT_BASES:
        tm, m = ck.terms(base)
        N, K = src[base + ".weight"].shape
        assert (m["mode"], m["packing"], m["terms"], m["group"], m["act"], tuple(m["shape"])) == (mode, fmt, terms, group, act, (N, K))
        assert len(tm) == terms
        for i, t in enumerate(tm):
            assert t.packed.dtype == torch.uint8 and tuple(t.packed.shape) == (N, -(-K // (5 if fmt == "tq1" else 4)))
            assert t.scale.dtype == sdt and tuple(t.scale.shape) == (N, -(-K // group))
            rec = m["stored"][f"{base}.tq{i}.packed"]
            assert tensor_sha256(t.packed) == rec["sha256"] and rec["file"] == "model-00001-of-00001.safetensors"
        lin = ck.linear(base)
        assert (lin.K, lin.fmt, lin.group, lin.act, lin.out_features) == (K, fmt, group, act, N)
    with pytest.raises(ValueError, match="mode 'A'"):
        ck.entry("layers.0.attn.wq")
    stacks, meta = ck.stack([f"layers.0.ffn.experts.{e}.w1" for e in range(2)], "cpu")
    assert meta == {"N": 16, "K": 200, "fmt": fmt, "group": group, "act": act, "terms": terms}
    assert len(stacks) == terms and tuple(stacks[0][0].shape) == (2, 16, 50 if fmt == "tq2" else 40)


def test_exported_terms_decode_to_the_source_weights():
    """What the stored bytes mean: the oracle's unpack x scales of the reference-written terms reconstruct the source weight
    to the error the reference's own test allows (tests/test_format.py:230-231: k = 2 on Gaussians < 0.3), padding included
    (K = 200: the last TQ1 byte holds no pad digits, the last TQ2 byte none either, the last scale group is 72 / 8 wide)."""
    src = _source()
    for name, fmt, group, bound in (("mode_c_tq1", "tq1", 128, 0.3), ("mode_d_tq2", "tq2", 64, 0.55)):
        ck = TernaryCheckpoint(EXPORTS / name)
        for base in EXPERT_BASES:
            tm, m = ck.terms(base)
            K = m["shape"][1]
            W = src[base + ".weight"].float().numpy()
            R = orc.dequantize([(t.packed.numpy(), t.scale.float().numpy()) for t in tm], K, group, fmt)
            err = np.linalg.norm(W - R) / np.linalg.norm(W)
            assert err < bound, (name, base, err)
            trits = orc.unpack(tm[0].packed.numpy(), fmt, K)
            assert set(np.unique(trits).tolist()) <= {-1, 0, 1}


def test_mode_d_export_equals_the_oracle_quantizer():
    """The reference's Mode D producer on general (Gaussian bf16) weights against oracle.absmean_ternary + pack: the stored
    scales and packed bytes are the oracle's, bit for bit - which pins the oracle's float32 summation order against
    torch's `abs().sum(-1)` on these rows (groups of 64 and a last group of 8)."""
    src = _source()
    ck = TernaryCheckpoint(EXPORTS / "mode_d_tq2")
    for base in EXPERT_BASES:
        tm, m = ck.terms(base)
        trits, scale = orc.absmean_ternary(src[base + ".weight"].float().numpy(), 64, "bf16")
        assert np.array_equal(tm[0].scale.float().numpy(), scale), base
        assert np.array_equal(tm[0].packed.numpy(), orc.pack(trits, "tq2")), base


@pytest.mark.gpu
def test_reference_written_checkpoints_run_on_the_gpu():
    """Both exports through `linear` on the device against the oracle on the decoded terms, and the Mode D export
    reproduced on the device from the source weights by bp_absmean_pack."""
    import deepseekternarized_amd as bp
    from deepseekternarized_amd.ternary.fit import packed_term

    src = _source()
    rng = np.random.default_rng(1)
    for name, fmt, group in (("mode_c_tq1", "tq1", 128), ("mode_d_tq2", "tq2", 64)):
        ck = TernaryCheckpoint(EXPORTS / name, verify=True)
        for base in EXPERT_BASES[:3]:
            lin = ck.linear(base)
            tm, m = ck.terms(base)
            K = m["shape"][1]
            x = orc.bf16_round(rng.standard_normal((3, K)).astype(np.float32))
            got = lin(torch.from_numpy(x).cuda().to(torch.bfloat16), out_dtype=torch.float32).cpu().numpy()
            want = orc.ternary_linear_ref(x, [(t.packed.numpy(), t.scale.float().numpy()) for t in tm], K, group, fmt, act=m["act"])
            assert np.linalg.norm(got - want) <= 1e-3 * np.linalg.norm(want), (name, base)
    ck = TernaryCheckpoint(EXPORTS / "mode_d_tq2")
    for base in EXPERT_BASES:
        tm, _ = ck.terms(base)
        term = packed_term(src[base + ".weight"].cuda(), 64, "tq2", scale_dtype=torch.bfloat16)
        assert torch.equal(term.packed.cpu(), tm[0].packed) and torch.equal(term.scale.cpu(), tm[0].scale), base
