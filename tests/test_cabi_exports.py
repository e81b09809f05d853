"""CPU-side checks of the boundary: the C-ABI libraries load and export every
symbol include/*.h declares (no compute calls), and the product path fails
loudly, with no CPU fallback, where there is no gfx950 device."""
import ctypes as C
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADERS = {"ojas_mi355x.h": ROOT / "ojas_amd" / "libojas_mi355x.so", "ojas_gpt.h": ROOT / "ojas_amd" / "libojas_gpt.so",
           "ojas_data.h": ROOT / "ojas_amd" / "libojas_data.so", "ojas_io.h": ROOT / "ojas_amd" / "libojas_io.so",
           "ojas_lora.h": ROOT / "ojas_amd" / "libojas_lora.so",
           "ojas_nanolab.h": ROOT / "ojas_amd" / "libojas_nanolab.so"}


def declared(header: Path):
    text = re.sub(r"/\*.*?\*/", "", header.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b((?:omx|ogpt|odata|oio|olora|onano)_\w+)\s*\(", text)))


@pytest.mark.parametrize("header", sorted(HEADERS))
def test_library_exports_every_declared_symbol(header):
    lib_path = HEADERS[header]
    assert lib_path.exists(), f"{lib_path} is not built; run __graft_entry__.build()"
    lib = C.CDLL(str(lib_path))
    names = declared(ROOT / "include" / header)
    assert len(names) >= 10
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_every_header_entry_cites_the_reference_interface_it_serves():
    text = (ROOT / "include" / "ojas_mi355x.h").read_text()
    for cite in ("backend.rs:1628", "backend.rs:1729", "backend.rs:1658", "backend.rs:2451", "backend.rs:2493",
                 "backend.rs:1610", "backend.rs:2468", "backend.rs:2480", "backend.rs:1466", "backend.rs:1514"):
        assert cite in text, cite


def test_no_device_means_a_loud_error_not_a_fallback():
    import torch  # only to learn whether this machine has a GPU

    if torch.cuda.is_available():
        pytest.skip("a GPU is present; the refusal path needs a machine without one")
    from ojas_amd.backend import DEVICE_LOST, MiBackend, OjasError

    with pytest.raises(OjasError) as e:
        MiBackend(0)
    assert e.value.code == DEVICE_LOST


def test_product_sources_never_reference_the_oracle():
    for path in list((ROOT / "ojas_amd").rglob("*")):
        if path.suffix in (".py", ".hip", ".cpp", ".h", ".hpp") or path.name == "Makefile":
            assert "oracle" not in path.read_text().lower(), path
