"""CPU checks of the drop-in boundary: the C-ABI library loads and exports exactly the
functions the public header declares (no compute calls here)."""
import ctypes
import os
import re

from muillm_amd import _lib


def test_library_is_built():
    assert os.path.exists(_lib.LIB_PATH), "run `make -C muillm_amd/csrc` first"


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    declared = _lib.declared_functions()
    assert len(declared) >= 6
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/muillm_amd.h but not exported"
        assert name in _lib._SIGNATURES, f"{name} has no ctypes signature in muillm_amd/_lib.py"
    for name in _lib._SIGNATURES:
        assert name in declared, f"{name} is bound in _lib.py but not declared in the header"


def test_signature_arity_matches_header():
    text = _lib.header_text()
    for name, (_, argtypes) in _lib._SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, text, flags=re.S)
        assert m, name
        args = m.group(1).strip()
        n = 0 if args in ("", "void") else len(args.split(","))
        assert n == len(argtypes), f"{name}: header has {n} parameters, ctypes binding {len(argtypes)}"


def test_no_framework_types_in_header():
    text = _lib.header_text()
    for banned in ("torch", "at::", "Tensor", "hipStream_t stream", "#include <hip"):
        assert banned not in text, banned


def test_product_header_holds_no_process_global_knobs():
    """The stateless product ABI and the sweep aids live in separate headers."""
    product = _lib.declared_functions(_lib.HEADER_PATH)
    aids = _lib.declared_functions(_lib.TUNE_HEADER_PATH)
    assert not [n for n in product if n.startswith("mui_tune") or n.startswith("mui_probe")]
    assert aids and all(n.startswith("mui_tune") or n.startswith("mui_probe") for n in aids)


def test_status_strings_and_version():
    lib = _lib.load()
    assert lib.mui_abi_version() == _lib.MUI_ABI_VERSION == 3
    assert _lib.status_string(0) == "ok"
    for code in (-1, -2, -3, -4, -5):
        assert _lib.status_string(code) not in ("ok", "unknown status")
    assert _lib.status_string(-99) == "unknown status"


def test_argument_validation_needs_no_gpu():
    """Null pointers and bad sizes are rejected on the host before any HIP call."""
    lib = _lib.load()
    assert lib.mui_linear(None, 0, None, 8, None, None, 0.0, None, None, None, None, 8, 8, 1) == -1
    assert lib.mui_rmsnorm(None, 0, None, None, 0.0, None, 1, 8) == -1
    assert lib.mui_gateup_silu(None, 0, None, None, 8, None, None, 0.0, None, 8, 8, 1) == -1
    assert lib.mui_device_info(0, None) == -1


def test_bench_refuses_more_than_one_gpu():
    """bench.py drives one GPU: any other --gpus value exits with a message (no GPU needed for this)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_tune_lock_freezes_the_knobs():
    """mui_tune_lock() is a one-way switch, so it is tried in a process of its own: before it the
    knobs answer, after it every one of them refuses and nothing changes (none of them touches a
    GPU, the library loads without one)."""
    import subprocess
    import sys

    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "from muillm_amd import _lib\n"
        "lib = _lib.load()\n"
        "assert lib.mui_tune_gemv(4, 2) == 0 and lib.mui_tune_gemv(0, 0) == 0\n"
        "assert lib.mui_tune_lock() == 0\n"
        "calls = [lib.mui_tune_gemv(4, 2), lib.mui_tune_int8(8, 2), lib.mui_tune_attention(8, 0, 0, 0),\n"
        "         lib.mui_tune_skinny(2, 0, 0), lib.mui_tune_packed_dot(1, 1), lib.mui_tune_prefill(0, 0),\n"
        "         lib.mui_tune_prefill_attention(0), lib.mui_tune_warm(256, 100, 0), lib.mui_tune_int8_quad(1, 0, 0, 0)]\n"
        "assert calls == [-2] * len(calls), calls\n"
        "print('locked')\n"
    ) % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))),)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "locked" in out.stdout, out.stderr
