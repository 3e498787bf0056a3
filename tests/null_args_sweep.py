"""Calls every bound entry point of Boat's API on libboat_amd.so with null pointers and zeros.

Run as a script in a process of its own (tests/test_null_arguments.py does): a missing NULL check would end the
process with a signal, which the parent sees as a negative return code.  The reference guards its entry points the
same way (`if (!tensor) return ...`), so a drop-in has to survive these calls too.
"""
import ctypes as C
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
import boat_amd.capi as capi  # noqa: E402


def main():
    api = capi.default_api()
    sigs = dict(capi._SIGS)
    sigs.update(capi._EXT_SIGS)
    for name, (_res, args) in sigs.items():
        vals = []
        for a in args:
            if a in (C.c_float, C.c_double):
                vals.append(0.0)
            elif a in (C.c_int, C.c_int32, C.c_int64, C.c_uint32, C.c_size_t, C.c_bool):
                vals.append(0)
            elif isinstance(a, type) and issubclass(a, C._CFuncPtr):
                vals.append(C.cast(None, a))
            else:
                vals.append(None)
        print(name, flush=True)
        getattr(api, name)(*vals)
    print("SURVIVED", len(sigs), flush=True)


if __name__ == "__main__":
    main()
