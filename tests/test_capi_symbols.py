"""The C-ABI library loads and exports every symbol that the headers under include/ declare (the boundary in
mimir_mi355x.h, the measurement aids in mimir_mi355x_measure.h). No compute call is made: this runs without a GPU."""
import os
import re

from mimir_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    inc = os.path.join(ROOT, "include")
    text = "".join(open(os.path.join(inc, f)).read() for f in sorted(os.listdir(inc)) if f.endswith(".h"))
    return set(re.findall(r"MI355X_API\s+[\w\s\*]+?\b(mi355x_\w+)\s*\(", text))


def test_header_and_binding_agree():
    declared = _declared()
    assert declared, "no declarations found"
    assert declared == set(capi.SYMBOLS), declared ^ set(capi.SYMBOLS)


def test_library_exports_every_symbol():
    lib = capi.load()
    for name in _declared():
        assert getattr(lib, name) is not None


def test_block_accounting_without_a_device():
    lib = capi.load()
    # backend/quant.go:24-59 with Q4_0 added
    assert [(lib.mi355x_block_size(d), lib.mi355x_block_bytes(d)) for d in (capi.Q8_0, capi.Q4_K, capi.Q6_K, capi.Q4_0)] == \
        [(32, 34), (256, 144), (256, 210), (32, 18)]
    assert lib.mi355x_bytes(capi.Q4_0, 4096 * 14336) == 4096 * 14336 // 32 * 18
    assert lib.mi355x_bytes(capi.Q8_0, 33) == -1 and lib.mi355x_bytes(capi.F32, 5) == 20 and lib.mi355x_bytes(0, 4) == -1


def test_every_tune_key_is_documented_and_every_documented_key_handled():
    """The keys mi355x_tune compares its argument with (capi.hip) are the keys that the header's comment on
    mi355x_tune names: a key added to one and not the other fails here."""
    src = open(os.path.join(ROOT, "mimir_amd", "csrc", "capi.hip")).read()
    body = src[src.index("mi355x_status mi355x_tune("):]
    handled = set(re.findall(r'strcmp\(key, "([^"]+)"\)', body))
    table = re.search(r'static const char\* keys\[\d+\] = \{([^}]*)\}', body)
    handled |= set(re.findall(r'"([^"]+)"', table.group(1))) if table else set()
    hdr = open(os.path.join(ROOT, "include", "mimir_mi355x.h")).read()
    documented = set(re.findall(r'"([a-z0-9_]+\.[a-zA-Z0-9_]+)"', hdr))
    assert handled and handled == documented, handled ^ documented
    lib = capi.load()
    assert lib.mi355x_tune(b"no.such_key", 1) != capi.OK  # and an unknown key is an error, without a device
