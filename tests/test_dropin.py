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


def test_the_sibling_modules_stage_with_their_binding_and_import_under_another_name(tmp_path):
    dropin.assemble(str(tmp_path))
    for folder, package_name, names in (("latent-attention", "latent_attention", ("attend", "prefill", "write", "partitions")),
                                        ("sparse-indexer", "sparse_indexer", ("scores", "topk", "select"))):
        root = os.path.join(str(tmp_path), folder)
        manifest = json.load(open(os.path.join(root, "kernel.json"), encoding="utf-8"))
        assert dropin.check_manifest(manifest, folder) == [] and manifest["package"] == package_name
        package = os.path.join(root, "torch-ext", package_name)
        assert sorted(os.listdir(package)) == ["__init__.py", "_pkv"]
        assert sorted(os.listdir(os.path.join(package, "_pkv"))) == ["__init__.py", "_abi.py", "libcrit_pkv.so"]
        name = package_name + "_staged_0123abcd"
        spec = importlib.util.spec_from_file_location(name, os.path.join(package, "__init__.py"),
                                                      submodule_search_locations=[package])
        module = importlib.util.module_from_spec(spec)
        sys.modules[name] = module
        try:
            spec.loader.exec_module(module)
            assert all(callable(getattr(module, n)) for n in names)
            assert os.path.join(package, "_pkv", "libcrit_pkv.so") in module._abi.candidates()
            assert module._abi.load().crit_pkv_abi_version() == module._abi.ABI_VERSION
        finally:
            for loaded in [n for n in sys.modules if n.startswith(name)]:
                sys.modules.pop(loaded, None)
