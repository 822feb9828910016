"""Loaders of the CPU checkers: test infrastructure, never part of the product path.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
`load_oracle()` opens oracle/liborc.so (the C restatement of the reference's CPU path);
`load_reference()` opens oracle/_ref/libqwen4_ref.so, the reference's own C sources compiled
where the reference tree is mounted, or returns None.  Both are typed with the same classes as
the shipped library (picoforge_amd.binding.MoeApi / HcApi), so callers drive all three alike.
"""
import ctypes as C
from pathlib import Path

from picoforge_amd.binding import HcApi, LibraryMissing, MoeApi

ORACLE_DIR = Path(__file__).resolve().parent


def _open(path):
    if not Path(path).exists():
        raise LibraryMissing(f"{path} is not built: run make -C oracle")
    return C.CDLL(str(path), mode=C.RTLD_LOCAL)


def load_oracle():
    lib = _open(ORACLE_DIR / "liborc.so")
    api = MoeApi(lib, moe_prefix="orc_moe_", private_prefix="orc_moe_", packed_prefix="orc_packed_")
    api.hc = HcApi(lib, prefix="orc_hc_")
    return api


def load_reference():
    path = ORACLE_DIR / "_ref" / "libqwen4_ref.so"
    if not path.exists():
        return None
    lib = _open(path)
    api = MoeApi(lib)
    api.hc = HcApi(lib)
    return api
