"""Child process of ``runtime.compile_source``: compiles one share of a large kernel set.

Run as a script (``python _compile_worker.py <library> <arch> <source file> <output file> [hiprtc options...]``, or
``<library> --version`` for the version of the hiprtc it would compile with);
it loads the C library directly and imports nothing of the package, so that it starts in a fraction of a second.
hiprtc needs no GPU and this process makes no other HIP call. ``OEQ_AMD_WORKER_PRELOAD`` lists the HIP runtime and
hiprtc files of the parent process (those of the torch wheel when torch is loaded there): they are loaded first, so
that the C library binds to them and this process compiles with the parent's compiler.
"""

import ctypes
import os
import sys


def main(argv) -> int:
    for path in filter(None, os.environ.get("OEQ_AMD_WORKER_PRELOAD", "").split(os.pathsep)):
        ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    lib = ctypes.CDLL(argv[0])
    if argv[1:] == ["--version"]:  # "<major>.<minor>.<patch>" of the ROCm release whose hiprtc this process compiles with
        with open("/proc/self/maps") as maps:
            files = [line.split()[-1] for line in maps if os.path.basename(line.split()[-1]).startswith("libamdhip64.so")]
        v = ctypes.c_int()
        if not files or ctypes.CDLL(files[0]).hipRuntimeGetVersion(ctypes.byref(v)) != 0:
            return 1
        print(f"{v.value // 10000000}.{v.value // 100000 % 100}.{v.value % 100000}")
        return 0
    _lib_file, arch, src_file, out_file, *opts = argv
    lib.oeq_jit_compile.restype = ctypes.c_int
    lib.oeq_jit_compile.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_char_p), ctypes.c_int,
                                    ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_size_t)]
    lib.oeq_last_error.restype = ctypes.c_char_p
    lib.oeq_free.argtypes = [ctypes.c_void_p]
    with open(src_file, "rb") as f:
        source = f.read()
    c_opts = (ctypes.c_char_p * len(opts))(*[o.encode() for o in opts])
    code, size = ctypes.c_void_p(), ctypes.c_size_t()
    rc = lib.oeq_jit_compile(source, arch.encode(), c_opts, len(opts), ctypes.byref(code), ctypes.byref(size))
    if rc:  # the compiler's words go to <output file>.err; exit status 3 says that the source is at fault
        with open(out_file + ".err", "wb") as f:
            f.write(lib.oeq_last_error() or b"")
        return 3
    with open(out_file, "wb") as f:
        f.write(ctypes.string_at(code.value, size.value))
    lib.oeq_free(code)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
