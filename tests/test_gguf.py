"""The GGUF reader and the drafter / target loaders (host code of the library; no GPU).

Pins: (1) the two fixture files of the reference's own CLI test (tests/golden/gguf/*.gguf, written by its tooling, not
by this repository's writer) must read back the facts its expected `qwen info` output states
(tests/golden/gguf/expected_info.json, extracted by tests/golden/make_gguf_expectations.py); (2) the malformed-file
cases of the reference's reader tests (crates/qwen-llm/src/gguf.rs:1822-1927, 2634-2712): overlap, rank 0 / 5, zero
dimension, unknown type, partial quant row, nested array, bad magic, bad version, truncated header, absurd counts;
(3) write -> read round trips of synthetic models through this repository's writer; (4) the drafter loader's rules
(crates/qwen-llm/src/loader.rs:832-1290) one by one."""
import json
import os
import struct

import numpy as np
import pytest

import qwen_llm_amd as dfl
from qwen_llm_amd import gguf as G

GOLD = os.path.join(os.path.dirname(__file__), "golden", "gguf")


@pytest.mark.parametrize("arch", ["qwen35", "qwen35moe"])
def test_reference_fixture_files_read_back_the_facts_of_the_reference_cli_baseline(arch):
    want = json.load(open(os.path.join(GOLD, "expected_info.json")))[arch]
    with dfl.GgufFile(os.path.join(GOLD, f"{arch}.gguf")) as g:
        assert g.architecture() == want["architecture"]
        assert g.tensor_count == want["tensors"]
        assert g.data_start == want["data_start"]
        names = [t.name for t in g.tensors()]
        assert [n for n in names if n.startswith("blk.0.")] == want["blk0_tensors"]
        for key, value in want["metadata"].items():
            assert g.get_u64(key) == value, key
        # every tensor lies inside the file, behind the header, on the alignment
        size = os.path.getsize(g.path)
        base = g.tensors()[0]._ptr - g.data_start
        for t in g.tensors():
            off = t._ptr - base
            assert off >= g.data_start and off % g.alignment == 0 and off + t.n_bytes <= size
            assert t.type == G.F32 and t.n_bytes == 4 * int(np.prod(t.shape))
        assert g.find("no.such.tensor") is None and g.get_u64("no.such.key") is None
        assert g.get_str("tokenizer.ggml.model") == "run-front-baseline"


# ---- malformed files (hand-assembled bytes) ----

def s(b):
    return struct.pack("<Q", len(b)) + b


def header(n_tensors, n_kv, version=3, magic=G.GGUF_MAGIC):
    return struct.pack("<IIQQ", magic, version, n_tensors, n_kv)


def tensor_info(name, shape, ttype, offset):
    return s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) + struct.pack("<IQ", ttype, offset)


def pad(b, a=32):
    return b + b"\0" * (-len(b) % a)


def open_bytes(tmp_path, data, name="f.gguf"):
    p = tmp_path / name
    p.write_bytes(data)
    return dfl.GgufFile(p)


def expect_format_error(tmp_path, data, fragment):
    with pytest.raises(dfl.DFlashError) as e:
        open_bytes(tmp_path, data)
    assert e.value.status == 12 and fragment in str(e.value), str(e.value)


def test_minimal_file_round_trip(tmp_path):
    data = pad(header(1, 1) + s(b"general.architecture") + struct.pack("<I", 8) + s(b"qwen35") +
               tensor_info(b"token_embd.weight", [4, 2], 0, 0)) + np.arange(8, dtype=np.float32).tobytes()
    with open_bytes(tmp_path, data) as g:
        assert g.architecture() == "qwen35" and g.tensor_count == 1 and g.kv_count == 1
        t = g.find("token_embd.weight")
        assert t.shape == (4, 2) and np.array_equal(t.f32(), np.arange(8, dtype=np.float32).reshape(2, 4))


def test_empty_tensor_table_may_end_unpadded(tmp_path):
    with open_bytes(tmp_path, header(0, 1) + s(b"k") + struct.pack("<II", 4, 7)) as g:
        assert g.tensor_count == 0 and g.get_u64("k") == 7


def test_malformed_files_are_rejected(tmp_path):
    f32x8 = np.zeros(8, np.float32).tobytes()
    expect_format_error(tmp_path, struct.pack("<I", 0x12345678) + b"\0" * 20, "magic")
    expect_format_error(tmp_path, header(0, 0, version=2), "version 2")
    expect_format_error(tmp_path, header(0, 0)[:12], "out-of-bounds")
    expect_format_error(tmp_path, header(10 ** 9, 0), "absurd tensor count")
    expect_format_error(tmp_path, header(0, 10 ** 9), "absurd kv count")
    # two tensors over the same bytes
    both = pad(header(2, 0) + tensor_info(b"a", [8], 0, 0) + tensor_info(b"b", [8], 0, 0)) + f32x8 * 2
    expect_format_error(tmp_path, both, "overlapping")
    expect_format_error(tmp_path, pad(header(1, 0) + s(b"a") + struct.pack("<I", 0) + struct.pack("<IQ", 0, 0)), "dimensions")
    expect_format_error(tmp_path, pad(header(1, 0) + tensor_info(b"a", [1, 1, 1, 1, 1], 0, 0)) + f32x8, "dimensions")
    expect_format_error(tmp_path, pad(header(1, 0) + tensor_info(b"a", [0, 2], 0, 0)) + f32x8, "zero-length")
    expect_format_error(tmp_path, pad(header(1, 0) + tensor_info(b"a", [1 << 31], 0, 0)) + f32x8, "exceeds")
    expect_format_error(tmp_path, pad(header(1, 0) + tensor_info(b"a", [8], 99, 0)) + f32x8, "unknown type")
    expect_format_error(tmp_path, pad(header(1, 0) + tensor_info(b"a", [100], 12, 0)) + b"\0" * 144, "multiple of the block size")
    nested = header(0, 1) + s(b"k") + struct.pack("<IIQ", 9, 9, 0)
    expect_format_error(tmp_path, nested, "nested")
    dup = header(0, 2) + (s(b"k") + struct.pack("<II", 4, 1)) * 2
    expect_format_error(tmp_path, dup, "duplicate metadata key")
    dupt = pad(header(2, 0) + tensor_info(b"a", [8], 0, 0) + tensor_info(b"a", [8], 0, 32)) + f32x8 * 2
    expect_format_error(tmp_path, dupt, "duplicate tensor name")
    expect_format_error(tmp_path, pad(header(1, 0) + tensor_info(b"a", [8], 0, 4)) + f32x8 * 2, "not aligned")
    expect_format_error(tmp_path, pad(header(1, 0) + tensor_info(b"a", [8], 0, 0)) + f32x8[:16], "past the end")
    expect_format_error(tmp_path, header(0, 1) + s(b"k") + struct.pack("<I", 13), "unknown metadata value type")
    expect_format_error(tmp_path, header(0, 1) + s(b"") + struct.pack("<II", 4, 1), "zero length")
    expect_format_error(tmp_path, header(0, 1) + s(b"\xff\xfe") + struct.pack("<II", 4, 1), "UTF-8")
    expect_format_error(tmp_path, header(0, 1) + s(b"general.alignment") + struct.pack("<II", 4, 0), "general.alignment")
    with pytest.raises(dfl.DFlashError) as e:
        dfl.GgufFile(tmp_path / "missing.gguf")
    assert e.value.status == 11


def test_metadata_getters_by_type(tmp_path):
    md = {"u8": (G._U8, 200), "i8": (G._I8, -3), "u16": (G._U16, 60000), "i32": (G._I32, 12), "u64": (G._U64, 1 << 40),
          "i64neg": (G._I64, -1), "f32": 1.5, "f64": (G._F64, 2.25), "flag": True, "name": "héllo",
          "ids": [1, 2, 3], "ids64": (G._I64, [4, 5]), "neg": (G._I64, [4, -5]), "flags": (G._BOOL, [True, False, True]),
          "fs": (G._F64, [0.5, 0.25]), "words": ["a", "bc"], "empty": (G._U32, [])}
    p = tmp_path / "kv.gguf"
    dfl.write_gguf(p, md, {})
    with dfl.GgufFile(p) as g:
        assert g.kv_count == len(md)
        assert (g.get_u64("u8"), g.get_u64("u16"), g.get_u64("i32"), g.get_u64("u64")) == (200, 60000, 12, 1 << 40)
        assert g.get_u64("i8") is None and g.get_u64("i64neg") is None  # negative: not a u64 (gguf.rs:514-517)
        assert g.get_u64("f32") is None and g.get_u64("name") is None
        assert g.get_f64("f32") == 1.5 and g.get_f64("f64") == 2.25 and g.get_f64("u8") is None
        assert g.get_bool("flag") is True and g.get_bool("u8") is None
        assert g.get_str("name") == "héllo" and g.get_str("u8") is None
        assert g.get_u64_array("ids") == [1, 2, 3] and g.get_u64_array("ids64") == [4, 5] and g.get_u64_array("empty") == []
        assert g.get_bool_array("flags") == [True, False, True] and g.get_f64_array("fs") == [0.5, 0.25]
        assert g.get_u64_array("absent") is None
        for key, getter in (("neg", g.get_u64_array), ("fs", g.get_u64_array), ("ids", g.get_bool_array), ("u8", g.get_u64_array),
                            ("words", g.get_f64_array)):
            with pytest.raises(dfl.DFlashError):
                getter(key)


def test_alignment_key_moves_the_data_start(tmp_path):
    p = tmp_path / "a.gguf"
    dfl.write_gguf(p, {"general.architecture": "x"}, {"t": np.arange(6, dtype=np.float32), "u": np.ones((2, 3), np.float32)},
                   alignment=256)
    with dfl.GgufFile(p) as g:
        assert g.alignment == 256 and g.data_start % 256 == 0
        assert np.array_equal(g.find("t").f32(), np.arange(6, dtype=np.float32))
        assert g.find("u").shape == (3, 2) and (g.find("u")._ptr - g.find("t")._ptr) == 256


# ---- drafter loader ----

TARGET = dict(hidden=256, vocab=512, n_layer=6)
D1 = dfl.DraftConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, block_size=16, n_taps=3, swa_window=128,
                     rope_theta=5e5, eps=float(np.float32(1e-5)))
D2 = dfl.DraftConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, block_size=8, n_taps=3, conv_kernel_size=2,
                     conv_group_size=64, selector_rank=64, selector_top_k=16)
IDS = [1, 3, 5]


def write_drafter(path, cfg, convention, w=None, md_edit=None, t_edit=None, swa=(False, True)):
    if not cfg.swa_window:
        swa = (False,) * cfg.n_layers
    w = w or dfl.synth_draft_weights(cfg, seed=2, wtype=dfl.TYPE_Q8_0, swa_layers=[i for i, x in enumerate(swa) if x],
                                     vocab=TARGET["vocab"], codebook_type=dfl.TYPE_Q8_0)
    md = G.draft_head_metadata(cfg, IDS, mask_token_id=511, swa_pattern=swa, convention=convention)
    t = G.draft_head_tensors(cfg, w, convention)
    if md_edit:
        md_edit(md)
    if t_edit:
        t_edit(t)
    dfl.write_gguf(path, md, t)
    return w


def load(path):
    with dfl.GgufFile(path) as g:
        cfg, w, ids, mask = dfl.open_dflash_drafter(g, TARGET["hidden"], TARGET["vocab"], TARGET["n_layer"])
        # copy out of the mapping before it goes away
        def own(x):
            return (x[0], np.array(x[1])) if isinstance(x, tuple) else (np.array(x) if isinstance(x, np.ndarray) else x)
        w = {k: ([{kk: own(vv) for kk, vv in L.items()} for L in v] if k == "layers" else own(v)) for k, v in w.items()}
    return cfg, w, ids, mask


def same_cfg(a, b):
    """Equal configurations; floats travel through the file as f32."""
    da, db = a.as_dict(), b.as_dict()
    return da.keys() == db.keys() and all(
        np.float32(da[k]) == np.float32(db[k]) if isinstance(da[k], float) else da[k] == db[k] for k in da)


def same_weights(a, b):
    if isinstance(a, tuple):
        return a[0] == b[0] and np.array_equal(np.asarray(a[1]).reshape(-1), np.asarray(b[1]).reshape(-1))
    if isinstance(a, np.ndarray):
        return np.array_equal(a, b)
    return a == b


@pytest.mark.parametrize("convention,cfg", [(1, D1), (2, D1), (2, D2)])
def test_drafter_file_round_trip(tmp_path, convention, cfg):
    p = tmp_path / "d.gguf"
    w = write_drafter(p, cfg, convention)
    got_cfg, got_w, ids, mask = load(p)
    assert same_cfg(got_cfg, cfg) and ids == IDS and mask == 511  # convention 2 stores ids + 1; post-block ids come back
    assert set(got_w) == set(w)
    for k in w:
        if k == "layers":
            for La, Lb in zip(w[k], got_w[k]):
                assert set(La) == set(Lb)
                for kk in La:
                    assert same_weights(La[kk], Lb[kk]), kk
        else:
            assert same_weights(w[k], got_w[k]), k


def expect_load_error(tmp_path, cfg, convention, fragment, **kw):
    p = tmp_path / "bad.gguf"
    write_drafter(p, cfg, convention, **kw)
    with pytest.raises(dfl.DFlashError) as e:
        load(p)
    assert fragment in str(e.value), str(e.value)
    return e.value


def test_drafter_loader_rules(tmp_path):
    P1, P2 = "dflash-draft", "dflash"
    expect_load_error(tmp_path, D1, 1, "unsupported architecture", md_edit=lambda m: m.update({"general.architecture": "qwen35"}))
    expect_load_error(tmp_path, D1, 1, f"{P1}.block_count", md_edit=lambda m: m.pop(f"{P1}.block_count"))
    expect_load_error(tmp_path, D1, 1, "does not fit 32 bits", md_edit=lambda m: m.update({f"{P1}.embedding_length": 1 << 33}))
    expect_load_error(tmp_path, D1, 1, "must equal the target's hidden size", md_edit=lambda m: m.update({f"{P1}.embedding_length": 128}))
    expect_load_error(tmp_path, D1, 1, "mask_token_id", md_edit=lambda m: m.update({f"{P1}.dflash.mask_token_id": 512}))
    expect_load_error(tmp_path, D1, 1, "past the target's", md_edit=lambda m: m.update({f"{P1}.dflash.target_layer_ids": [1, 3, 6]}))
    expect_load_error(tmp_path, D1, 1, "n_target_features mismatch", md_edit=lambda m: m.update({f"{P1}.dflash.n_target_features": 512}))
    expect_load_error(tmp_path, D1, 1, "must equal block_count", md_edit=lambda m: m.update({f"{P1}.attention.sliding_window_pattern": (G._BOOL, [True])}))
    expect_load_error(tmp_path, D1, 1, "sliding_window is missing or 0", md_edit=lambda m: m.pop(f"{P1}.attention.sliding_window"))
    expect_load_error(tmp_path, D1, 1, "must be a multiple of", md_edit=lambda m: m.update({f"{P1}.attention.head_count_kv": 3}))
    expect_load_error(tmp_path, D1, 1, "layer_norm_rms_epsilon", md_edit=lambda m: m.update({f"{P1}.attention.layer_norm_rms_epsilon": 0.0}))
    expect_load_error(tmp_path, D1, 1, "must be nonzero", md_edit=lambda m: m.update({f"{P1}.dflash.block_size": 0}))
    expect_load_error(tmp_path, D1, 1, "exceeds the cap", md_edit=lambda m: m.update({f"{P1}.dflash.block_size": 5000}))
    expect_load_error(tmp_path, D1, 1, "missing tensor blk.1.attn_k_norm.weight", t_edit=lambda t: t.pop("blk.1.attn_k_norm.weight"))
    expect_load_error(tmp_path, D1, 1, "expected shape [256, 128], got [256, 256]",
                      t_edit=lambda t: t.update({"blk.0.attn_k.weight": t["blk.0.attn_q.weight"]}))
    # the other convention's names are not looked up
    expect_load_error(tmp_path, D1, 2, "missing tensor fc.weight", t_edit=lambda t: t.update({"dflash_fc.weight": t.pop("fc.weight")}))
    expect_load_error(tmp_path, D1, 2, "cannot capture layer input 0", md_edit=lambda m: m.update({f"{P2}.target_layers": [0, 2, 4]}))
    # DFlash-2: selector_hidden.weight makes the four keys and every conv / selector tensor mandatory
    expect_load_error(tmp_path, D2, 2, "dflash.selector_rank", md_edit=lambda m: m.pop("dflash.selector_rank"))
    expect_load_error(tmp_path, D2, 2, "must divide embedding_length", md_edit=lambda m: m.update({"dflash.conv_group_size": 48}))
    expect_load_error(tmp_path, D2, 2, "exceeds the cap", md_edit=lambda m: m.update({"dflash.conv_kernel_size": 9}))
    expect_load_error(tmp_path, D2, 2, "missing tensor blk.0.ffn_conv_base", t_edit=lambda t: t.pop("blk.0.ffn_conv_base"))
    expect_load_error(tmp_path, D2, 2, "missing tensor selector_successor.weight", t_edit=lambda t: t.pop("selector_successor.weight"))
    e = expect_load_error(tmp_path, D1, 1, "must be F32",
                          t_edit=lambda t: t.update({"output_norm.weight": (G.F16, (256,), np.zeros(512, np.uint8))}))
    assert e.status == 2
    # defaults: rope base 1e7, eps 1e-6, causal true when the keys are absent (loader.rs:956-975)
    p = tmp_path / "defaults.gguf"
    write_drafter(p, D1, 1, md_edit=lambda m: [m.pop(f"{P1}.{k}") for k in ("rope.freq_base", "attention.layer_norm_rms_epsilon", "attention.causal")])
    cfg = load(p)[0]
    assert cfg.rope_theta == 1e7 and cfg.eps == np.float32(1e-6) and cfg.causal == 1
    # a drafter without the selector tensor is a DFlash-1 head even under the "dflash" convention
    p = tmp_path / "v2_plain.gguf"
    write_drafter(p, D1, 2)
    assert load(p)[0].selector_rank == 0


# ---- target loader ----

def test_target_file_round_trip_dense_and_moe(tmp_path):
    dense = dfl.ModelConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, vocab=512)
    moe = dfl.ModelConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=0, vocab=512, n_expert=8, n_expert_used=2,
                          ffn_expert=256, ffn_shared=256)
    for cfg in (dense, moe):
        w = dfl.synth_target_weights(cfg, seed=4)
        p = tmp_path / f"t{cfg.n_expert}.gguf"
        dfl.write_gguf(p, G.target_metadata(cfg), G.target_tensors(cfg, w))
        with dfl.GgufFile(p) as g:
            got_cfg, got_w = dfl.open_target(g)
            assert same_cfg(got_cfg, cfg)
            assert same_weights(w["token_embd"], got_w["token_embd"]) and same_weights(w["output"], got_w["output"])
            for La, Lb in zip(w["layers"], got_w["layers"]):
                assert set(La) == set(Lb)
                for kk in La:
                    assert same_weights(La[kk], Lb[kk]), kk
    # tied embeddings: no output.weight -> the embedding serves as the output head (loader.rs:445-452)
    w = dfl.synth_target_weights(dense, seed=4)
    p = tmp_path / "tied.gguf"
    dfl.write_gguf(p, G.target_metadata(dense), G.target_tensors(dense, w, tied=True))
    with dfl.GgufFile(p) as g:
        _, got_w = dfl.open_target(g)
        assert same_weights(got_w["output"], w["token_embd"])
    # the hybrid architectures of the reference's fixtures are refused, not misread
    with dfl.GgufFile(os.path.join(GOLD, "qwen35.gguf")) as g:
        with pytest.raises(dfl.DFlashError) as e:
            dfl.open_target(g)
        assert "unsupported architecture" in str(e.value)


# ---- split (multi-shard) models: the cases of the reference's own tests (gguf.rs:2223-2640) ----

def split_shard(path, no, count, total, tensors, extra=None):
    md = dict(extra or {})
    md.update({"split.no": (G._U16, no), "split.count": (G._U16, count), "split.tensors.count": (G._I32, total)})
    G.write_gguf(path, md, tensors)


def one(v):
    return np.full(1, v, np.float32)


def expect_split_error(path, status, fragment):
    with pytest.raises(dfl.DFlashError) as e:
        dfl.GgufFile(path)
    assert e.value.status == status and fragment in str(e.value), str(e.value)


def test_split_model_opens_from_its_first_shard(tmp_path):
    """opens_split_gguf_from_first_shard (gguf.rs:2223): two shards, one tensor each at the same shard-local offset."""
    first, second = tmp_path / "model-00001-of-00002.gguf", tmp_path / "model-00002-of-00002.gguf"
    split_shard(first, 0, 2, 2, {"a": one(1.0)}, {"general.architecture": "qwen35"})
    split_shard(second, 1, 2, 2, {"b": one(2.0)}, {"general.architecture": "other"})
    with dfl.GgufFile(first) as g:
        assert g.shard_count == 2 and g.tensor_count == 2
        assert [t.name for t in g.tensors()] == ["a", "b"]            # shard order
        assert g.find("a").f32()[0] == 1.0 and g.find("b").f32()[0] == 2.0
        assert g.architecture() == "qwen35"                             # the first shard's metadata is the model's


def test_write_split_gguf_round_trip(tmp_path):
    rng = np.random.default_rng(0)
    shards = [{"a": rng.standard_normal((3, 8)).astype(np.float32)}, {},
              {"b": rng.standard_normal(64).astype(np.float32), "c": one(7.0)}]
    paths = G.write_split_gguf(tmp_path / "m", {"general.architecture": "qwen35moe", "k": 5}, shards)
    assert [p.rsplit("/", 1)[1] for p in paths] == ["m-00001-of-00003.gguf", "m-00002-of-00003.gguf", "m-00003-of-00003.gguf"]
    with dfl.GgufFile(paths[0]) as g:
        assert g.shard_count == 3 and g.tensor_count == 3 and g.get_u64("k") == 5
        for sh in shards:
            for name, a in sh.items():
                assert np.array_equal(g.find(name).f32(), a)
    # a single file reports one shard
    G.write_gguf(tmp_path / "single.gguf", {"split.count": (G._U16, 1)}, {"a": one(1.0)})
    with dfl.GgufFile(tmp_path / "single.gguf") as g:
        assert g.shard_count == 1 and g.tensor_count == 1


def test_split_model_with_unpadded_empty_first_shard(tmp_path):
    """opens_split_gguf_with_unpadded_empty_first_shard (gguf.rs:2323): a metadata-only first shard may end at its header."""
    first, second = tmp_path / "model-00001-of-00002.gguf", tmp_path / "model-00002-of-00002.gguf"
    kv = (s(b"split.no") + struct.pack("<IH", 2, 0) + s(b"split.count") + struct.pack("<IH", 2, 2) +
          s(b"split.tensors.count") + struct.pack("<Ii", 5, 1))
    first.write_bytes(header(0, 3) + kv)
    split_shard(second, 1, 2, 1, {"only": one(3.0)})
    with dfl.GgufFile(first) as g:
        assert g.shard_count == 2 and g.tensor_count == 1 and g.find("only").f32()[0] == 3.0


def test_split_model_rejections(tmp_path, monkeypatch):
    a, b = {"a": one(1.0)}, {"b": one(2.0)}

    def pair(name):
        d = tmp_path / name
        d.mkdir()
        return d / "model-00001-of-00002.gguf", d / "model-00002-of-00002.gguf"

    # rejects_opening_nonfirst_split (:2375)
    first, second = pair("nonfirst")
    split_shard(second, 1, 2, 2, b)
    expect_split_error(second, 12, "must be loaded with the first split")
    # rejects_missing_split_sibling (:2395): an I/O error, not a format error
    first, second = pair("missing")
    split_shard(first, 0, 2, 2, a)
    expect_split_error(first, 11, "cannot open")
    # rejects_bad_split_suffix (:2415)
    split_shard(tmp_path / "model.gguf", 0, 2, 1, a)
    expect_split_error(tmp_path / "model.gguf", 12, "invalid split file name")
    split_shard(tmp_path / "-00001-of-00002.gguf", 0, 2, 1, a)   # a suffix and nothing before it
    monkeypatch.chdir(tmp_path)
    expect_split_error("-00001-of-00002.gguf", 12, "invalid split file: ")
    # rejects_wrong_split_no (:2435)
    first, second = pair("wrong_no")
    split_shard(first, 0, 2, 2, a)
    split_shard(second, 0, 2, 2, b)
    expect_split_error(first, 12, "invalid split file idx: 0")
    # rejects_wrong_split_count (:2468)
    first, second = pair("wrong_count")
    split_shard(first, 0, 2, 2, a)
    split_shard(second, 1, 3, 2, b)
    expect_split_error(first, 12, "invalid split count: 3")
    # a sibling with another total
    first, second = pair("wrong_total")
    split_shard(first, 0, 2, 2, a)
    split_shard(second, 1, 2, 3, b)
    expect_split_error(first, 12, "invalid split tensor count: 3")
    # rejects_duplicate_tensor_names_across_splits (:2501)
    first, second = pair("dup")
    split_shard(first, 0, 2, 2, a)
    split_shard(second, 1, 2, 2, a)
    expect_split_error(first, 12, "duplicated across GGUF splits")
    # rejects_split_tensor_count_mismatch (:2534): fewer tensors than declared
    first, second = pair("short")
    split_shard(first, 0, 2, 3, a)
    split_shard(second, 1, 2, 3, b)
    expect_split_error(first, 12, "3 tensors expected but 2 found")
    # rejects_split_tensor_count_overrun_while_merging (:2567): more than declared, caught before the merge
    first, second = pair("over")
    split_shard(first, 0, 2, 1, a)
    split_shard(second, 1, 2, 1, b)
    expect_split_error(first, 12, "declare 1 tensors but at least 2")
    # rejects_absurd_split_count_before_allocating_paths (:2600)
    G.write_gguf(tmp_path / "absurd-00001-of-02000.gguf", {"split.no": (G._U16, 0), "split.count": (G._U16, 2000),
                                                          "split.tensors.count": (G._I32, 1)}, a)
    expect_split_error(tmp_path / "absurd-00001-of-02000.gguf", 12, "exceeds cap 1024")
    # rejects_absurd_split_tensor_count_before_allocating_table (:2617)
    G.write_gguf(tmp_path / "big-00001-of-00002.gguf", {"split.no": (G._U16, 0), "split.count": (G._U16, 2),
                                                       "split.tensors.count": (G._U64, 10 ** 9)}, a)
    expect_split_error(tmp_path / "big-00001-of-00002.gguf", 12, "split.tensors.count 1000000000")
    # the first shard without its number or its total
    G.write_gguf(tmp_path / "nono-00001-of-00002.gguf", {"split.count": (G._U16, 2), "split.tensors.count": (G._I32, 1)}, a)
    expect_split_error(tmp_path / "nono-00001-of-00002.gguf", 12, 'missing "split.no"')
    G.write_gguf(tmp_path / "nototal-00001-of-00002.gguf", {"split.count": (G._U16, 2), "split.no": (G._U16, 0)}, a)
    expect_split_error(tmp_path / "nototal-00001-of-00002.gguf", 12, 'missing "split.tensors.count"')


def test_drafter_loads_from_a_split_model(tmp_path):
    """The loader sees one tensor table whichever shard holds a tensor: a drafter written over three shards reads
    back the same configuration and weights as from one file."""
    w = write_drafter(tmp_path / "one.gguf", D2, 2)
    md = G.draft_head_metadata(D2, IDS, mask_token_id=511, swa_pattern=(False,) * D2.n_layers, convention=2)
    t = G.draft_head_tensors(D2, w, 2)
    names = list(t)
    paths = G.write_split_gguf(tmp_path / "drafter", md, [{n: t[n] for n in names[i::3]} for i in range(3)])
    with dfl.GgufFile(paths[0]) as g:
        assert g.shard_count == 3 and g.tensor_count == len(names)
    cfg1, w1, ids1, mask1 = load(tmp_path / "one.gguf")
    cfg3, w3, ids3, mask3 = load(paths[0])
    assert same_cfg(cfg1, cfg3) and ids1 == ids3 and mask1 == mask3
    for k in w1:
        if k == "layers":
            for La, Lb in zip(w1[k], w3[k]):
                for kk in La:
                    assert same_weights(La[kk], Lb[kk]), kk
        else:
            assert same_weights(w1[k], w3[k]), k
