"""ctypes view of include/nerva_hip_api.h.

The Structures are built by parsing the header, so the Python side can never
drift from the C ABI: field order, widths and pointer-ness come from the one
source of truth the C++ code is compiled against.
"""
import ctypes as C
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(os.path.dirname(_HERE), "include", "nerva_hip_api.h")
LIBRARY = os.path.join(_HERE, "libnerva_hip.so")

_SCALARS = {
    "int32_t": C.c_int32, "uint32_t": C.c_uint32, "uint64_t": C.c_uint64, "int64_t": C.c_int64,
    "uint16_t": C.c_uint16, "uint8_t": C.c_uint8, "float": C.c_float, "char": C.c_char, "int": C.c_int,
    "void": None,
}


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _parse_structs(text):
    structs = {}
    opaque = set(re.findall(r"typedef struct (\w+) \1;", text))
    for name in opaque:
        structs[name] = type(name, (C.Structure,), {})
    for m in re.finditer(r"typedef struct (\w+) \{(.*?)\} \1;", text, flags=re.S):
        name, body = m.group(1), m.group(2)
        fields = []
        for decl in body.split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            decl = decl.replace("const ", "")
            base, rest = decl.split(" ", 1)
            for item in rest.split(","):
                item = item.strip()
                stars = item.count("*")
                ident = item.replace("*", "").strip()
                arr = re.match(r"(\w+)\[(\d+)\]$", ident)
                if base in _SCALARS:
                    ctype = _SCALARS[base]
                elif base in structs:
                    ctype = structs[base]
                else:
                    raise ValueError("unknown type %s in %s" % (base, name))
                if stars:
                    # data pointers are passed as raw addresses (device or host)
                    ctype = C.POINTER(ctype) if (ctype is not None and isinstance(ctype, type)
                                                 and issubclass(ctype, C.Structure)) else C.c_void_p
                    for _ in range(stars - 1):
                        ctype = C.POINTER(ctype)
                if arr:
                    ident, count = arr.group(1), int(arr.group(2))
                    ctype = ctype * count
                fields.append((ident, ctype))
        structs[name] = type(name, (C.Structure,), {"_fields_": fields})
    return structs


def _parse_functions(text):
    body = text
    out = {}
    for m in re.finditer(r"\b(int|uint64_t)\s+(nerva_hip_\w+)\s*\(([^;{]*?)\)\s*;", body, flags=re.S):
        out[m.group(2)] = (m.group(1), " ".join(m.group(3).split()))
    return out


_TEXT = _strip_comments(open(HEADER).read())
STRUCTS = _parse_structs(_TEXT)
FUNCTIONS = _parse_functions(_TEXT)
globals().update(STRUCTS)
CONSTANTS = {m.group(1): int(m.group(2).rstrip("u"), 0)
             for m in re.finditer(r"#define (NERVA_HIP_\w+) (-?\w+)", _TEXT) if m.group(2)[0].isdigit()}
globals().update(CONSTANTS)


def _arg_type(arg):
    arg = arg.replace("const ", "").strip()
    if arg == "void":
        return None
    stars = arg.count("*")
    base = arg.split()[0].replace("*", "")
    if stars == 0:
        return _SCALARS[base]
    if base in STRUCTS:
        t = C.POINTER(STRUCTS[base])
        for _ in range(stars - 1):
            t = C.POINTER(t)
        return t
    if stars == 2:
        return C.POINTER(C.c_void_p)
    if base == "int32_t":
        return C.POINTER(C.c_int32)
    return C.c_void_p


def declared_symbols():
    return sorted(FUNCTIONS)


class MissingLibrary(RuntimeError):
    pass


_lib = None


def load():
    """Load libnerva_hip.so and attach argtypes/restype for every declared entry point.

    Fails loudly when the HIP library has not been built: there is no CPU fallback.
    """
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY):
        raise MissingLibrary("%s is missing: build it with `python -m nerva_amd.build` "
                             "(hipcc, gfx950). There is no fallback path." % LIBRARY)
    lib = C.CDLL(LIBRARY)
    for name, (ret, args) in FUNCTIONS.items():
        fn = getattr(lib, name)  # AttributeError here = header/library mismatch
        fn.restype = C.c_int if ret == "int" else C.c_uint64
        types = [_arg_type(a) for a in args.split(",")] if args.strip() else []
        fn.argtypes = [t for t in types if t is not None]
    _lib = lib
    return lib
