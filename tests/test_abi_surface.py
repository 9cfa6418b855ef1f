"""CPU-side checks of the boundary: the shared library loads without a GPU and
exports every symbol the header declares; nothing in the product package touches
the oracle."""
import os
import re

from cavs_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    l = hip.lib()
    names = hip.declared_symbols()
    assert len(names) >= 45
    missing = [n for n in names if not hasattr(l, n)]
    assert not missing, missing
    assert l.cavs_abi_version() >= 1
    bound = set(hip._SIGS) | set(hip._NOCHECK)
    assert set(names) == bound, sorted(set(names) ^ bound)


def test_header_cites_the_reference_for_every_entry_group():
    text = open(hip.HEADER).read()
    assert len(re.findall(r"cavs/(backend|midend|util)/[a-z0-9_./]+:\d+", text)) >= 20


def test_product_never_touches_the_oracle():
    bad = []
    for base in ("cavs_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            if "build" in dirpath.split(os.sep) or "__pycache__" in dirpath:
                continue
            for f in files:
                if f.endswith((".py", ".hip", ".h", ".cc", ".cpp")):
                    src = open(os.path.join(dirpath, f), errors="ignore").read()
                    if re.search(r"pyoracle|cavs_oracle|libcavs_oracle|or_model_step|oracle/", src):
                        bad.append(os.path.join(dirpath, f))
    assert not bad, bad
