"""The Rust `-sys` crate shipped as source (qwen-llm_amd/rust/dflash-hip-sys) is generated from the C header: it must
be what the header generates today and declare exactly the functions the library exports.  (No Rust toolchain exists
in this environment, so the crate is not compiled here.)"""
import importlib.util
import os
import re

import qwen_llm_amd as dfl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _gen():
    spec = importlib.util.spec_from_file_location("gen_sys", os.path.join(ROOT, "qwen-llm_amd", "rust", "gen_sys.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_bindings_are_current_and_complete():
    gen = _gen()
    text = open(gen.OUT).read()
    assert text == gen.generate(), "run: python qwen-llm_amd/rust/gen_sys.py"
    assert set(re.findall(r"pub fn (\w+)\(", text)) == set(dfl.declared_symbols())
    assert "_private" in text and "*mut *mut dflash_ctx" in text and "name: *mut *const c_char" in text


def test_struct_layouts_match_the_ctypes_mirror():
    """Field counts and order of the structs both mirrors declare (the ctypes one is exercised against the library by
    every other test, so agreement here is what can be checked of the Rust one without a compiler)."""
    from qwen_llm_amd import binding, gguf, model

    text = open(_gen().OUT).read()
    structs = {m.group(1): re.findall(r"pub (\w+): ", m.group(2))
               for m in re.finditer(r"pub struct (\w+) \{\n(.*?)\n\}", text, flags=re.S)}
    pairs = {"dflash_model_cfg": model.ModelCfgC, "dflash_layer": model.LayerC, "dflash_model": model.ModelC,
             "dflash_draft_cfg": model.DraftCfgC, "dflash_draft_layer": model.DraftLayerC, "dflash_draft_head": model.DraftHeadC,
             "dflash_adaptive_state": model.AdaptiveStateC, "dflash_gguf_tensor": gguf.GgufTensorC,
             "dflash_gguf_draft_layer": gguf.GgufDraftLayerC, "dflash_gguf_draft_head": gguf.GgufDraftHeadC,
             "dflash_target_shape": gguf.TargetShapeC, "dflash_accept_decision": binding.AcceptDecisionC}
    for name, c in pairs.items():
        want = [f[0] for f in c._fields_]
        got = [g[:-1] if g.endswith("_") and g[:-1] in want else g for g in structs[name]]
        assert got == want, name
