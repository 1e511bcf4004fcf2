"""Prints the C# P/Invoke declarations of every function include/prad_hip.h declares.

    python -m parallelreverseautodiff_amd.pinvoke            # the PradHip class body, one DllImport per entry point

The reference is C# (ParallelReverseAutoDiff.RMAD); its operations would bind libprad_hip.so through these
declarations.  They are generated from the header so that they cannot fall behind it.
"""
import os
import re

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "prad_hip.h")

# C parameter type -> C# parameter type.  Device pointers and handles travel as IntPtr; arrays of handles / row
# pointers as IntPtr[]; out-parameters as `out`.
_TYPES = [
    (r"const prad_buf_t\s*\*", "IntPtr[]"),
    (r"prad_buf_t\s*\*", "out IntPtr"),
    (r"prad_buf_t", "IntPtr"),
    (r"const void\s*\*\s*const\s*\*", "IntPtr[]"),
    (r"void\s*\*\s*const\s*\*", "IntPtr[]"),
    (r"void\s*\*\*", "out IntPtr"),
    (r"const void\s*\*", "IntPtr"),
    (r"void\s*\*", "IntPtr"),
    (r"const int64_t\s*\*", "long[]"),
    (r"int64_t\s*\*", "out long"),
    (r"int32_t\s*\*", "out int"),
    (r"const (double|float)\s*\*", "IntPtr"),
    (r"(double|float)\s*\*", "IntPtr"),   # device memory; the host out-parameters are listed in _HOST_OUT
    (r"int64_t", "long"),
    (r"int32_t", "int"),
    (r"double", "double"),
]
# (function, parameter) pairs whose float* / double* points at a host variable that the call fills in.
_HOST_OUT = {("prad_event_elapsed_ms", "ms"): "out float"}
_RESERVED = {"out", "in", "ref", "params", "base", "lock", "event", "object", "string"}


def prototypes(header_text=None):
    """[(return type, name, [(C type, parameter name)])] in header order."""
    text = header_text if header_text is not None else open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    out = []
    for ret, name, params in re.findall(r"(int32_t|void\s*\*|const char\s*\*)\s+(prad_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        plist = []
        params = " ".join(params.split())
        if params and params != "void":
            for p in params.split(","):
                p = p.strip()
                m = re.match(r"(.*?)(\w+)$", p)
                plist.append((m.group(1).strip(), m.group(2)))
        out.append((" ".join(ret.split()), name, plist))
    return out


def csharp_type(ctype, function=None, parameter=None):
    if (function, parameter) in _HOST_OUT:
        return _HOST_OUT[(function, parameter)]
    for pattern, cs in _TYPES:
        if re.fullmatch(pattern, ctype):
            return cs
    raise ValueError("no C# mapping for parameter type %r" % ctype)


def declaration(ret, name, params):
    cs_ret = "int" if ret == "int32_t" else "IntPtr"
    args = []
    for ctype, pname in params:
        cs = csharp_type(ctype, name, pname)
        if pname in _RESERVED:
            pname = "@" + pname
        args.append("%s %s" % (cs, pname))
    return "[DllImport(Lib)] public static extern %s %s(%s);" % (cs_ret, name, ", ".join(args))


def declarations():
    return [declaration(*p) for p in prototypes()]


if __name__ == "__main__":
    print("\n".join(declarations()))
