"""CPU-side checks: the C-ABI library loads and exports every declared symbol."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header, folder="include"):
    text = open(os.path.join(ROOT, folder, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:dq8|tao_ral|disc_ral)_[a-z0-9_]+)\s*\(", text)))


def test_exports_every_declared_symbol():
    from bladedisc_amd import _lib
    L = _lib.lib()
    headers = [h for h in os.listdir(os.path.join(ROOT, "include")) if h.endswith(".h")]
    assert headers
    total = 0
    for h in headers:
        for name in _declared(h):
            assert hasattr(L, name), "%s declared in %s but not exported" % (name, h)
            total += 1
    assert total >= 10


def test_exports_the_test_hooks():
    """The variant-forcing entry points and the MFMA layout probe are declared in a
    tests-only header, not in the product ABI."""
    from bladedisc_amd import _lib
    L = _lib.lib()
    hooks = _declared("dq8_test_hooks.h", "tests")
    assert "dq8_qgemm_variant" in hooks and "dq8_mfma_probe" in hooks
    for name in hooks:
        assert hasattr(L, name), name
    public = set()
    for h in os.listdir(os.path.join(ROOT, "include")):
        public |= set(_declared(h))
    assert not public & set(hooks)


def test_variant_table_and_version():
    from bladedisc_amd import kernels
    names = kernels.variant_names()
    assert names[0] == "generic" and len(names) >= 4


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """No CPU fallback: without the built library every operator raises."""
    import pytest
    from bladedisc_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libdisc_q8_ral.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.lib()
    from bladedisc_amd import kernels
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        kernels.variant_names()
