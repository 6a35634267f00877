"""The names the reference's own modules, runners and tests import from the modules this package
mirrors (tests/golden/import_surface.json, written from the reference's sources by
tests/golden/make_import_surface.py: fast_decode.py:232-243, blockwise_decode.py:23-43,
obkv_fast.py:38-46, run_latency.py:38-46, tests/test_blockwise_rdkv.py:14-20, ...): each is
present under the same module name in ``rdkv_amd`` with the same parameters in the same order, so
that aliasing ``obkv_accel.<module>`` to ``rdkv_amd.<module>`` keeps every import working."""
import dataclasses
import importlib
import inspect
import json
import os

import pytest

SURFACE = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "import_surface.json")))

# Triton device functions of the reference (pointer, stride and constexpr parameters, callable
# from inside a Triton kernel only): here they are host-callable tile helpers, so only the names
# match.
DEVICE_HELPERS = {"dequant_2bit_v_tile", "dequant_4bit_v_tile", "dequant_8bit_v_tile", "unpack_2bit_k_codes_kt",
                  "unpack_4bit_k_codes_kt", "unpack_8bit_k_codes_kt"}
# Names of the reference's top-level obkv_fast.py that are outside the decode-attention / packing
# path: model loading, the prefill and its eviction, the tensor-expression decode loops, dataset
# and file helpers of the benchmark runners.
OUT_OF_SCOPE = {
    "obkv_fast": {"DEFAULT_MODEL_PATH", "_streaming_prefill_and_pack", "detach_past_key_values", "ensure_dir",
                  "evict_past_key_values", "greedy_decode_pt", "greedy_decode_pt_with_perhead_masks", "load_json",
                  "load_model_and_tokenizer", "middle_truncate_token_ids", "patch_llama31_rope_compat",
                  "prefill_last_token", "prepare_past_key_values_for_model", "run_obkv", "set_determinism"},
}


def _cases():
    for module, names in sorted(SURFACE.items()):
        for name, entry in sorted(names.items()):
            yield module, name, entry


@pytest.mark.parametrize("module,name,entry", list(_cases()), ids=[f"{m}.{n}" for m, n, _ in _cases()])
def test_reference_import_resolves_here(module, name, entry):
    short = module.split(".")[-1]
    ours = importlib.import_module("rdkv_amd." + short)
    definition = entry["definition"]
    if definition is None:
        # the reference imports a name its own module does not define (decode_hook.py:42,54 ask
        # triton_k_kernel for k_dequant_qk_dot[_ref]); there is nothing to mirror
        assert module == "obkv_accel.triton_k_kernel" and name.startswith("k_dequant_qk_dot")
        return
    if name in OUT_OF_SCOPE.get(short, ()):
        assert not hasattr(ours, name), f"{short}.{name} exists: take it off the out-of-scope list"
        return
    assert hasattr(ours, name), f"rdkv_amd.{short} lacks {name} (imported by {entry['importers']})"
    obj = getattr(ours, name)
    if definition["kind"] == "function":
        assert callable(obj)
        if name in DEVICE_HELPERS:
            return
        params = list(inspect.signature(obj).parameters.values())
        names_here = [p.name for p in params]
        ref_pos = definition["params"]
        assert names_here[:len(ref_pos)] == ref_pos, f"{short}.{name}: parameters {names_here} vs the reference's {ref_pos}"
        for kw in definition["kwonly"]:
            assert kw in names_here, f"{short}.{name}: keyword {kw} missing"
        # anything this package adds is optional
        extra = [p for p in params[len(ref_pos):] if p.name not in definition["kwonly"]]
        assert all(p.default is not inspect.Parameter.empty or p.kind in (p.VAR_KEYWORD, p.VAR_POSITIONAL)
                   for p in extra), f"{short}.{name}: extra required parameters {[p.name for p in extra]}"
    elif definition["kind"] == "class":
        assert inspect.isclass(obj)
        if definition["fields"] and dataclasses.is_dataclass(obj):
            here = [f.name for f in dataclasses.fields(obj)]
            assert here[:len(definition["fields"])] == definition["fields"], f"{short}.{name}: fields {here}"


def test_every_mirrored_module_is_listed():
    """The modules the integration recipe aliases are the ones the reference imports from."""
    assert {m.split(".")[-1] for m in SURFACE} == {
        "bitpack", "blockwise_decode", "fast_decode", "packing", "triton_dequant_utils", "triton_k_kernel",
        "triton_rope", "triton_v_kernel", "trizone_decompress", "obkv_fast"}
