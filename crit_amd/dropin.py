"""Assembles the folders crit's kernel loader expects for the kernel ids `paged-kv-attention`, `latent-attention` and
`sparse-indexer`:

    <dest>/paged-kv-attention/kernel.json
    <dest>/paged-kv-attention/torch-ext/paged_kv_attention/{__init__.py, _abi.py, libcrit_pkv.so}
    <dest>/latent-attention/kernel.json
    <dest>/latent-attention/torch-ext/latent_attention/{__init__.py, _pkv/{__init__.py, _abi.py, libcrit_pkv.so}}
    <dest>/sparse-indexer/kernel.json
    <dest>/sparse-indexer/torch-ext/sparse_indexer/{__init__.py, _pkv/...}

    python -m crit_amd.dropin <dest>          # then: export CRIT_KERNEL_PATH=<dest>  (or replace crit's own folder)

crit's loader copies torch-ext/<package>/ into its cache and imports it under another name with relative imports
working (reference kernels/crit_kernels/build.py:864-880, 932-954); the package therefore carries the built library
beside its Python files and imports nothing outside itself.
"""
import json
import os
import shutil
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PACKAGE = os.path.join(HERE, "paged_kv_attention")
LEVELS = ("declared", "exact", "row-exact", "repeatable")


def check_manifest(manifest, folder_name):
    """The rules of the loader this manifest must pass (reference build.py:77-91, exactness.py:127-169): schema, an id
    equal to the folder's name, a level for every structure, `exact` exactly where bits_of names another structure
    whose root is row-exact or declared."""
    problems = []
    if manifest.get("schema") != "crit-kernel-v1":
        problems.append("schema is not crit-kernel-v1")
    if manifest.get("id") != folder_name:
        problems.append("id differs from the folder's name")
    structures = manifest.get("structures", {})
    for name, s in structures.items():
        level = s.get("exactness")
        if level not in LEVELS:
            problems.append(f"{name}: no exactness level")
        if (level == "exact") != ("bits_of" in s):
            problems.append(f"{name}: exact comes with bits_of and only with it")
        if "bits_of" in s:
            root = structures.get(s["bits_of"], {})
            if root.get("exactness") not in ("row-exact", "declared"):
                problems.append(f"{name}: bits_of names no row-exact structure")
    return problems


def assemble(dest, library=None):
    """Write the drop-in folder under dest; returns its path. The library must be built (python -m crit_amd.build)."""
    library = library or os.path.join(HERE, "lib", "libcrit_pkv.so")
    if not os.path.exists(library):
        raise FileNotFoundError(f"{library}: build it first (python -m crit_amd.build)")
    root = os.path.join(dest, "paged-kv-attention")
    package = os.path.join(root, "torch-ext", "paged_kv_attention")
    os.makedirs(package, exist_ok=True)
    manifest = json.load(open(os.path.join(PACKAGE, "kernel.json"), encoding="utf-8"))
    problems = check_manifest(manifest, "paged-kv-attention")
    if problems:
        raise ValueError("; ".join(problems))
    shutil.copy(os.path.join(PACKAGE, "kernel.json"), os.path.join(root, "kernel.json"))
    for name in ("__init__.py", "_abi.py"):
        shutil.copy(os.path.join(PACKAGE, name), os.path.join(package, name))
    shutil.copy(library, os.path.join(package, "libcrit_pkv.so"))
    for folder, module in SIBLINGS.items():
        assemble_sibling(dest, folder, module, library)
    return root


SIBLINGS = {"latent-attention": "latent_attention", "sparse-indexer": "sparse_indexer"}


def assemble_sibling(dest, folder, module, library):
    """The folder of a kernels module that launches through the paged-KV package's binding (its launch helper, its
    ctypes mirrors, the one library): the loader imports a staged package under another name with nothing beside it,
    so the package carries a copy of that binding as its subpackage `_pkv` and imports it from there."""
    source = os.path.join(HERE, module)
    manifest = json.load(open(os.path.join(source, "kernel.json"), encoding="utf-8"))
    problems = check_manifest(manifest, folder)
    if problems:
        raise ValueError("; ".join(problems))
    root = os.path.join(dest, folder)
    package = os.path.join(root, "torch-ext", module)
    binding = os.path.join(package, "_pkv")
    os.makedirs(binding, exist_ok=True)
    shutil.copy(os.path.join(source, "kernel.json"), os.path.join(root, "kernel.json"))
    text = open(os.path.join(source, "__init__.py"), encoding="utf-8").read()
    if "from ..paged_kv_attention import" not in text:
        raise ValueError(f"{module}: no import of the paged-KV binding to stage")
    with open(os.path.join(package, "__init__.py"), "w", encoding="utf-8") as f:
        f.write(text.replace("from ..paged_kv_attention import", "from ._pkv import"))
    for name in ("__init__.py", "_abi.py"):
        shutil.copy(os.path.join(PACKAGE, name), os.path.join(binding, name))
    shutil.copy(library, os.path.join(binding, "libcrit_pkv.so"))
    return root


if __name__ == "__main__":
    if len(sys.argv) != 2:
        sys.exit(__doc__)
    print(assemble(sys.argv[1]))
