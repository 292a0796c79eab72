"""Child process of ``runtime.compile_source``: compiles one share of a large kernel set.

Run as a script (``python _compile_worker.py <library> <arch> <source file> <output file> [hiprtc options...]``);
it loads the C library directly and imports nothing of the package, so that it starts in a fraction of a second.
hiprtc needs no GPU and this process makes no other HIP call. ``OEQ_AMD_WORKER_PRELOAD`` lists the HIP runtime and
hiprtc files of the parent process (those of the torch wheel when torch is loaded there): they are loaded first, so
that the C library binds to them and this process compiles with the parent's compiler.
"""

import ctypes
import os
import sys


def main(argv) -> int:
    lib_file, arch, src_file, out_file, *opts = argv
    for path in filter(None, os.environ.get("OEQ_AMD_WORKER_PRELOAD", "").split(os.pathsep)):
        ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    lib = ctypes.CDLL(lib_file)
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
    if rc:
        sys.stderr.write((lib.oeq_last_error() or b"").decode(errors="replace") + "\n")
        return 1
    with open(out_file, "wb") as f:
        f.write(ctypes.string_at(code.value, size.value))
    lib.oeq_free(code)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
