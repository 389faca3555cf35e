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


def test_the_product_library_exports_its_headers_and_nothing_else():
    """The variant-forcing entry points and the MFMA layout probe are declared in a tests-only
    header and live in libdisc_q8_testhooks.so; libdisc_q8_ral.so exports the C ABI of
    include/*.h and no other symbol."""
    import subprocess
    from bladedisc_amd import _lib
    L, H = _lib.lib(), _lib.hooks()
    hooks = _declared("dq8_test_hooks.h", "tests")
    assert "dq8_qgemm_variant" in hooks and "dq8_mfma_probe" in hooks
    public = set()
    for h in os.listdir(os.path.join(ROOT, "include")):
        public |= set(_declared(h))
    assert not public & set(hooks)
    for name in hooks:
        assert hasattr(H, name), name
        assert not hasattr(L, name), name + " is exported by the product library"
    for name in public:
        assert hasattr(H, name), name
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True,
                         text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    extra = {e for e in exported if e not in public and e != "kMlirLoweredEntry"}
    assert not extra, sorted(extra)[:20]


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
    monkeypatch.setattr(_lib, "_hooks", None)
    monkeypatch.setattr(_lib, "HOOKS_LIB_PATH", str(tmp_path / "libdisc_q8_testhooks.so"))
    from bladedisc_amd import kernels
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        kernels.variant_names()
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        kernels.qlinear_f32_fused_max_rows(768, 768)
