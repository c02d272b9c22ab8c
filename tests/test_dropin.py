"""The drop-in folder for crit's kernel loader assembles, its manifest passes the loader's rules, and the staged
package imports under another name with only relative imports (as the loader imports it)."""
import importlib.util
import json
import os
import sys

from crit_amd import dropin


def test_the_manifest_passes_the_loaders_rules():
    manifest = json.load(open(os.path.join(dropin.PACKAGE, "kernel.json"), encoding="utf-8"))
    assert dropin.check_manifest(manifest, "paged-kv-attention") == []
    assert manifest["package"] == "paged_kv_attention" and manifest["language"] == "triton" and "cuda" not in manifest
    for name in ("write", "split", "window", "merge", "prefill"):
        assert manifest["structures"][name]["exactness"] == "row-exact"
    assert dropin.check_manifest(dict(manifest, id="other"), "paged-kv-attention")
    broken = json.loads(json.dumps(manifest))
    del broken["structures"]["fused"]["bits_of"]
    assert dropin.check_manifest(broken, "paged-kv-attention")


def test_the_staged_package_imports_under_another_name(tmp_path):
    root = dropin.assemble(str(tmp_path))
    package = os.path.join(root, "torch-ext", "paged_kv_attention")
    assert sorted(os.listdir(package)) == ["__init__.py", "_abi.py", "libcrit_pkv.so"]
    name = "paged_kv_attention_staged_0123abcd"
    spec = importlib.util.spec_from_file_location(name, os.path.join(package, "__init__.py"),
                                                  submodule_search_locations=[package])
    module = importlib.util.module_from_spec(spec)
    sys.modules[name] = module
    try:
        spec.loader.exec_module(module)
        assert module.MAX_COLUMNS == 64 and callable(module.attend)
        assert os.path.join(package, "libcrit_pkv.so") in module._abi.candidates()
        lib = module._abi.load()
        assert lib.crit_pkv_abi_version() == module._abi.ABI_VERSION
    finally:
        sys.modules.pop(name, None)
        sys.modules.pop(name + "._abi", None)
