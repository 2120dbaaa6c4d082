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


def test_adapter_names_only_what_the_sys_crate_declares():
    """The DFlashDecoder-shaped adapter (qwen-llm_amd/rust/dflash-hip) is source only: every `sys::` name it uses must
    be declared by the generated -sys crate (functions = the library's exports), every struct field it touches must
    exist, and it must offer the reference's decoder surface (metal_dflash.rs:8328-8555, 17257-17415)."""
    gen = _gen()
    sys_text = open(gen.OUT).read()
    adapter = open(os.path.join(ROOT, "qwen-llm_amd", "rust", "dflash-hip", "src", "lib.rs")).read()
    declared_fns = set(re.findall(r"pub fn (\w+)\(", sys_text))
    declared_types = set(re.findall(r"pub struct (\w+)", sys_text))
    declared_consts = set(re.findall(r"pub const (\w+):", sys_text))
    used = set(re.findall(r"\bsys::(\w+)", adapter))
    assert used, "adapter does not use the sys crate"
    unknown = used - declared_fns - declared_types - declared_consts
    assert not unknown, f"adapter names symbols the sys crate does not declare: {sorted(unknown)}"
    assert (used & declared_fns) <= set(dfl.declared_symbols())
    # argument counts of the calls match the declarations
    for name in used & declared_fns:
        decl = re.search(r"pub fn %s\((.*?)\)(?: -> [\w*: ]+)?;" % name, sys_text).group(1)
        n_decl = 0 if not decl.strip() else decl.count(",") + 1
        for m in re.finditer(r"sys::%s\(" % name, adapter):
            depth, i, n_args, any_arg = 1, m.end(), 0, False
            while depth:
                ch = adapter[i]
                if ch in "([{":
                    depth += 1
                elif ch in ")]}":
                    depth -= 1
                elif ch == "," and depth == 1:
                    n_args += 1
                elif ch == "|" and depth == 1:  # closure bars inside an argument
                    pass
                if not ch.isspace() and depth:
                    any_arg = True
                i += 1
            n_args = n_args + 1 if any_arg else 0
            assert n_args == n_decl, f"{name}: adapter passes {n_args} arguments, declaration has {n_decl}"
    # struct fields the adapter reads
    fields = {m.group(1): set(re.findall(r"pub (\w+): ", m.group(2)))
              for m in re.finditer(r"pub struct (\w+) \{\n(.*?)\n\}", sys_text, flags=re.S)}
    for struct, names in {"dflash_draft_cfg": ["block_size", "selector_rank", "selector_top_k"],
                          "dflash_draft_head": ["cfg", "selector_predecessor", "selector_successor"],
                          "dflash_model": ["cfg"], "dflash_model_cfg": ["vocab"],
                          "dflash_step_result": ["decision"], "dflash_accept_decision": ["err_row"],
                          "dflash_weighted_candidate": ["token", "pad", "weight"]}.items():
        for f in names:
            assert f in fields[struct], f"{struct}.{f}"
    for method in ("pub fn new(", "pub fn packed_verify(", "pub fn packed_verify_with_logits(",
                   "pub fn restore_after_partial_accept(", "pub fn draft_block(", "pub fn draft_block_sampled(",
                   "pub fn spec_step("):
        assert method in adapter, method
