"""ctypes binding of liboeq_amd.so (the C ABI in include/oeq_amd.h) plus the
kernel cache: source -> hiprtc code object -> loaded kernel set.

Stands in for the reference's extension loader and kernel cache
(openequivariance/openequivariance/_torch/extlib/__init__.py:36-204 and
extension/torch_core.hpp:180-270). There is no CPU fallback: if the shared
library is missing every entry point raises.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import subprocess
import threading
from pathlib import Path
from typing import Dict, List, Optional, Sequence, Tuple

_PKG_DIR = Path(__file__).resolve().parent
_REPO_DIR = _PKG_DIR.parent
_LIB_PATH = _PKG_DIR / "liboeq_amd.so"
_SRC_PATH = _PKG_DIR / "csrc" / "oeq_amd.cpp"
_INCLUDE_DIR = _REPO_DIR / "include"

DEFAULT_ARCH = "gfx950"

# Flags for every device compile. Packed-FP32 instruction selection is turned
# off on purpose (scalar v_fma_f32 only).
HIPRTC_OPTIONS = [
    "-O3",
    "--std=c++17",
    "-ffp-contract=fast",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

ROLE_TP_FORWARD = 0
ROLE_TP_BACKWARD = 1
ROLE_CONV_FORWARD = 2
ROLE_CONV_BACKWARD = 3
ROLE_CONV_FIXUP_BACKWARD = 4
ROLE_SEGMENT_PTR = 5
ROLE_FILL_ZERO = 6
ROLE_TP_BACKWARD_WREDUCE = 7
ROLE_SEGMENT_SUM = 8
ROLE_GROUP_COUNT = 9
ROLE_GROUP_SCAN = 10
ROLE_GROUP_SCATTER = 11
ROLE_GROUP_ORDER = 12
ROLE_DOUBLE_BACKWARD_A = 13
ROLE_DOUBLE_BACKWARD_B = 14
ROLE_ORDER_HOP = 15
ROLE_HUB_COUNT = 16
ROLE_HUB_FILL = 17
ROLE_CONV_FIXUP_FORWARD = 18
ROLE_CONV_BACKWARD_DX = 19

CONV_ATOMIC, CONV_SORTED, CONV_GROUPED = 0, 1, 2
DX_TERMS, DX_ATOMIC, DX_ARRIVAL, DX_SENDER_WALK = 0, 1, 2, 3
ABI_VERSION = 6


class OeqError(RuntimeError):
    pass


class DeviceProps(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 256),
        ("arch", ctypes.c_char * 64),
        ("wave_size", ctypes.c_int32),
        ("compute_units", ctypes.c_int32),
        ("lds_per_block", ctypes.c_int32),
        ("max_threads_per_block", ctypes.c_int32),
        ("clock_khz", ctypes.c_int32),
        ("l2_bytes", ctypes.c_int32),
        ("total_mem", ctypes.c_int64),
    ]


class _KernelDesc(ctypes.Structure):
    _fields_ = [
        ("role", ctypes.c_int32),
        ("kernel_name", ctypes.c_char_p),
        ("block_threads", ctypes.c_uint32),
        ("units_per_block", ctypes.c_uint32),
        ("max_blocks", ctypes.c_uint32),
        ("grid_multiple", ctypes.c_uint32),
    ]


class _ProblemDims(ctypes.Structure):
    _fields_ = [
        ("L1_dim", ctypes.c_int64),
        ("L2_dim", ctypes.c_int64),
        ("L3_dim", ctypes.c_int64),
        ("weight_numel", ctypes.c_int64),
        ("elem_size", ctypes.c_int32),
        ("shared_weights", ctypes.c_int32),
        ("deterministic", ctypes.c_int32),
        ("wpartial_per_block", ctypes.c_int32),
        ("dx_mode", ctypes.c_int32),
        ("n_chunks", ctypes.c_int32),
        ("order_hops", ctypes.c_int32),
        ("hub_limit", ctypes.c_int32),
    ]


def build_library(verbose: bool = False) -> Path:
    """Compile csrc/oeq_amd.cpp into liboeq_amd.so next to this file."""
    # the library carries one device-side object (the scratch array of oeq_conv_forward_static), so it is
    # compiled for the target architecture, with the device flags every kernel here is compiled with
    # built under a temporary name and moved into place, so that a process loading the library while
    # another one rebuilds it never maps a half-written file
    tmp = _LIB_PATH.with_name(f"{_LIB_PATH.name}.tmp{os.getpid()}")
    cmd = [
        "hipcc", "-O2", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={DEFAULT_ARCH}",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", f"-I{_INCLUDE_DIR}",
        str(_SRC_PATH), "-o", str(tmp), "-lhiprtc",
    ]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise OeqError(f"building liboeq_amd.so failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, _LIB_PATH)
    if verbose:
        print(" ".join(cmd).replace(str(tmp), str(_LIB_PATH)))
    return _LIB_PATH


_lib = None
_lib_lock = threading.Lock()

_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_SZ = ctypes.c_size_t

EXPORTS = {
    "oeq_get_device_props": (ctypes.c_int, [ctypes.c_int, ctypes.POINTER(DeviceProps)]),
    "oeq_jit_compile": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_char_p),
                                       ctypes.c_int, ctypes.POINTER(_P), ctypes.POINTER(_SZ)]),
    "oeq_free": (None, [_P]),
    "oeq_kernels_create": (ctypes.c_int, [_P, _SZ, ctypes.POINTER(_ProblemDims), ctypes.POINTER(_KernelDesc),
                                          ctypes.c_int, ctypes.POINTER(_P)]),
    "oeq_kernels_destroy": (None, [_P]),
    "oeq_tp_forward": (ctypes.c_int, [_P, _I64, _P, _P, _P, _P, _P]),
    "oeq_tp_backward": (ctypes.c_int, [_P, _I64, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "oeq_tp_backward_workspace_bytes": (_SZ, [_P, _I64]),
    "oeq_conv_forward": (ctypes.c_int, [_P, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "oeq_conv_forward_workspace_bytes": (_SZ, [_P, _I64, _I64]),
    "oeq_conv_forward_static": (ctypes.c_int, [_P, _I64, _I64, _P, _P, _P, _P, _P, _P, _P]),
    "oeq_static_scratch_bytes": (_SZ, []),
    "oeq_conv_backward": (ctypes.c_int, [_P, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "oeq_conv_backward_workspace_bytes": (_SZ, [_P, _I64, _I64]),
    "oeq_conv_double_backward_workspace_bytes": (_SZ, [_P, _I64, _I64]),
    "oeq_conv_index_bytes": (_SZ, [_P, _I64, _I64, ctypes.c_int]),
    "oeq_conv_index_build": (ctypes.c_int, [_P, _I64, _I64, _P, _P, _P, ctypes.c_int, _P, _SZ, _P]),
    "oeq_conv_forward_indexed": (ctypes.c_int, [_P, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _SZ, ctypes.c_int, _P, _SZ,
                                                _P]),
    "oeq_conv_forward_scratch_bytes": (_SZ, [_P, _I64, _I64]),
    "oeq_conv_index_piece": (ctypes.c_int, [_P, _I64, _I64, ctypes.c_int, ctypes.c_int, ctypes.POINTER(_SZ),
                                            ctypes.POINTER(_SZ)]),
    "oeq_conv_backward_indexed": (ctypes.c_int, [_P, _I64, _I64] + [_P] * 10 + [_P, _SZ, ctypes.c_int, _P, _SZ, _P]),
    "oeq_conv_backward_scratch_bytes": (_SZ, [_P, _I64, _I64]),
    "oeq_conv_double_backward_indexed": (ctypes.c_int, [_P, _I64, _I64] + [_P] * 14 + [_P, _SZ, _P, _SZ, _P]),
    "oeq_conv_double_backward_scratch_bytes": (_SZ, [_P, _I64, _I64]),
    "oeq_has_double_backward": (ctypes.c_int, [_P]),
    "oeq_tp_double_backward": (ctypes.c_int, [_P, _I64] + [_P] * 12 + [_SZ, _P]),
    "oeq_tp_double_backward_workspace_bytes": (_SZ, [_P, _I64]),
    "oeq_conv_double_backward": (ctypes.c_int, [_P, _I64, _I64] + [_P] * 15 + [_SZ, _P]),
    "oeq_segment_sum": (ctypes.c_int, [_P, _I64, _I64, _I64, _P, _P, _P, _P, _P, _SZ, _P]),
    "oeq_segment_sum_workspace_bytes": (_SZ, [_P, _I64]),
    "oeq_grouped_sum": (ctypes.c_int, [_P, _I64, _I64, _I64, _P, _P, _P, _P, _SZ, _P]),
    "oeq_grouped_sum_workspace_bytes": (_SZ, [_P, _I64, _I64]),
    "oeq_kernel_timing_enable": (ctypes.c_int, [_P, ctypes.c_int]),
    "oeq_kernel_timing_collect": (ctypes.c_int, [_P, ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                                                 ctypes.POINTER(_I64)]),
    "oeq_last_error": (ctypes.c_char_p, []),
    "oeq_abi_version": (ctypes.c_int, []),
}


def lib_path() -> Path:
    return _LIB_PATH


def _stale() -> bool:
    """The built library is older than the sources it is made from."""
    built = _LIB_PATH.stat().st_mtime
    return any(src.exists() and src.stat().st_mtime > built for src in (_SRC_PATH, _INCLUDE_DIR / "oeq_amd.h"))


def load_library():
    """Load liboeq_amd.so. It is built first when no built file exists or the file is older than its
    sources; a library whose ABI version is not the one this module binds is refused (kernel argument
    lists are positional, so a mismatch would mean wrong pointers on the GPU rather than an error)."""
    global _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not _LIB_PATH.exists() or _stale():
            build_library()
        lib = ctypes.CDLL(str(_LIB_PATH))
        try:
            lib.oeq_abi_version.restype = ctypes.c_int
            found = lib.oeq_abi_version()
        except AttributeError:
            found = None
        if found != ABI_VERSION:
            raise OeqError(f"{_LIB_PATH} has ABI version {found}, this package needs {ABI_VERSION}: "
                           "rebuild it (python -c 'import __graft_entry__ as g; g.build()' at the repository root)")
        for name, (res, args) in EXPORTS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
        return lib


def _check(rc: int, what: str):
    if rc != 0:
        msg = load_library().oeq_last_error()
        raise OeqError(f"{what} failed ({rc}): {msg.decode(errors='replace') if msg else ''}")


def device_props(device: int = 0) -> DeviceProps:
    props = DeviceProps()
    _check(load_library().oeq_get_device_props(device, ctypes.byref(props)), "oeq_get_device_props")
    return props


# ---------------------------------------------------------------------------
# compile + on-disk cache of code objects
# ---------------------------------------------------------------------------


def cache_dir() -> Path:
    d = os.environ.get("OEQ_AMD_CACHE_DIR")
    path = Path(d) if d else _PKG_DIR / "_kcache"
    path.mkdir(parents=True, exist_ok=True)
    return path


def source_hash(source: str, arch: str = DEFAULT_ARCH, options: Optional[Sequence[str]] = None) -> str:
    h = hashlib.sha256()
    h.update(arch.encode())
    h.update("\0".join(options if options is not None else HIPRTC_OPTIONS).encode())
    h.update(source.encode())
    return h.hexdigest()[:24]


def _compile_one(source: str, arch: str, opts: Sequence[str]) -> bytes:
    lib = load_library()
    c_opts = (ctypes.c_char_p * len(opts))(*[o.encode() for o in opts])
    code = _P()
    size = _SZ()
    rc = lib.oeq_jit_compile(source.encode(), arch.encode(), c_opts, len(opts), ctypes.byref(code), ctypes.byref(size))
    _check(rc, "oeq_jit_compile")
    try:
        return ctypes.string_at(code.value, size.value)
    finally:
        lib.oeq_free(code)


# Large kernel sets are compiled side by side. hiprtc compiles one program at a time per process (eight threads
# take as long as one: 94 s against 98 s for the 327 kernels of a 128-channel, l <= 3 shared-weight 'uvw' problem),
# so the kernels are dealt out to that many child processes, each of which compiles the set's shared declarations
# and device functions with its share of the kernels (the same problem on 8 cores: 16 s). The code objects travel
# as one pack, which oeq_kernels_create takes apart (layout: see pack_code).
PACK_MAGIC = b"OEQPACK1"
PARALLEL_MIN_BYTES = 256 * 1024  # kernel text below which a set is compiled in this process (a few seconds)
_WORKER_PATH = _PKG_DIR / "_compile_worker.py"


def compile_jobs() -> int:
    """Child processes a large kernel set is compiled in (``OEQ_AMD_COMPILE_JOBS``; 1 = never split)."""
    env = os.environ.get("OEQ_AMD_COMPILE_JOBS")
    if env:
        return max(1, int(env))
    return max(1, min(16, os.cpu_count() or 1))


def split_kernels(source: str) -> Tuple[str, List[str]]:
    """(everything but the kernels, [kernel definitions]) of a generated module. A kernel definition runs from a
    line that starts with ``extern "C" __global__`` to the next line that is a lone closing brace (the emitters
    indent everything inside a definition); one inside a ``namespace x {`` ... ``}  // namespace x`` pair of such
    lines is returned wrapped in that namespace, whose other members stay where they are."""
    common, kernels, cur, space = [], [], None, None
    for ln in source.split("\n"):
        if cur is not None:
            cur.append(ln)
            if ln == "}":
                text = "\n".join(cur)
                kernels.append(f"namespace {space} {{\n{text}\n}}" if space else text)
                cur = None
            continue
        if ln.startswith('extern "C" __global__'):
            cur = [ln]
            continue
        if ln.startswith("namespace ") and ln.rstrip().endswith("{"):
            space = ln[len("namespace "):].rstrip()[:-1].strip()
        elif space and ln.startswith("}") and f"namespace {space}" in ln:
            space = None
        common.append(ln)
    if cur is not None:  # not laid out like a generated module: nothing to split
        return source, []
    return "\n".join(common), kernels


def pack_code(blobs: Sequence[bytes]) -> bytes:
    """Several code objects as one: ``PACK_MAGIC``, a uint64 count, that many uint64 sizes, then the objects in
    order, each from the next multiple of 64 bytes (little endian; what oeq_kernels_create accepts in place of
    a single code object)."""
    import struct
    out = bytearray(PACK_MAGIC + struct.pack(f"<Q{len(blobs)}Q", len(blobs), *[len(b) for b in blobs]))
    for b in blobs:
        out += b"\0" * (-len(out) % 64)
        out += b
    return bytes(out)


def unpack_code(blob: bytes) -> List[bytes]:
    """The code objects of what compile_source returned (one, unless it is a pack)."""
    import struct
    if not blob.startswith(PACK_MAGIC):
        return [blob]
    (count,) = struct.unpack_from("<Q", blob, 8)
    sizes = struct.unpack_from(f"<{count}Q", blob, 16)
    out, at = [], 16 + 8 * count
    for n in sizes:
        at += -at % 64
        out.append(blob[at:at + n])
        at += n
    return out


def _kernel_descriptors(blob: bytes) -> Dict[str, bytes]:
    """{kernel name: its 64-byte kernel descriptor} (the objects ``<name>.kd`` of an amdhsa code object) of the
    kernels in what compile_source returned."""
    import struct
    out: Dict[str, bytes] = {}
    for elf in unpack_code(blob):
        shoff, = struct.unpack_from("<Q", elf, 0x28)
        shentsize, shnum = struct.unpack_from("<HH", elf, 0x3A)
        sections = [struct.unpack_from("<IIQQQQIIQQ", elf, shoff + i * shentsize) for i in range(shnum)]
        for _name, kind, _flags, _addr, off, size, link, _info, _align, entsize in sections:
            if kind != 2:  # SHT_SYMTAB
                continue
            str_off = sections[link][4]
            for at in range(off, off + size, entsize):
                st_name, _st_info, _other, st_shndx, st_value, st_size = struct.unpack_from("<IBBHQQ", elf, at)
                end = elf.index(b"\0", str_off + st_name)
                name = elf[str_off + st_name:end].decode()
                if not name.endswith(".kd") or st_size != 64 or not 0 < st_shndx < shnum:
                    continue
                sec = sections[st_shndx]
                start = sec[4] + st_value - sec[3]
                out[name[:-3]] = elf[start:start + 64]
    return out


def kernel_resources(blob: bytes) -> Dict[str, Tuple[int, int]]:
    """{kernel name: (bytes of LDS, bytes of scratch memory per lane)} of the kernels in what compile_source
    returned, from the kernel descriptors (whose first two 32-bit words are group_segment_fixed_size and
    private_segment_fixed_size). A kernel that the compiler could not fit into its register budget has a
    non-zero scratch size."""
    import struct
    return {name: struct.unpack_from("<II", kd, 0) for name, kd in _kernel_descriptors(blob).items()}


def kernel_registers(blob: bytes) -> Dict[str, int]:
    """{kernel name: vector registers a lane of it is allocated} (architectural and accumulation registers
    together, in the granules of eight that gfx90a and later allocate: bits 5:0 of compute_pgm_rsrc1, the
    32-bit word at byte 48 of the kernel descriptor, hold the granule count minus one). A SIMD's 512 registers
    per lane divided by this number is how many waves of the kernel it holds."""
    import struct
    return {name: ((struct.unpack_from("<I", kd, 48)[0] & 0x3F) + 1) * 8
            for name, kd in _kernel_descriptors(blob).items()}


def _loaded_rocm_libraries() -> Dict[str, str]:
    """{name: file} of the HIP runtime and hiprtc this process has loaded."""
    wanted, found = ("libamdhip64", "libhiprtc"), {}
    try:
        with open("/proc/self/maps") as maps:
            for line in maps:
                path = line.split()[-1]
                for name in wanted:
                    if os.path.basename(path).startswith(name + ".so"):
                        found.setdefault(name, path)
    except OSError:
        pass
    return {n: found[n] for n in wanted if n in found}


def _compile_parallel(source: str, arch: str, opts: Sequence[str], jobs: int, own_compiler: bool = True,
                      always: bool = False) -> Optional[bytes]:
    """The pack of a large module's code objects (one plain code object when it is compiled as one share), or
    None when the module is small or has a single kernel and ``always`` is not set, or a child process could not
    be run or failed (the caller then compiles in this process, which also reports a compile error in full).
    ``own_compiler``: the children load this process's HIP libraries first, else they take the system's."""
    import sys
    import tempfile
    common, kernels = split_kernels(source)
    small = len(kernels) < 2 or sum(map(len, kernels)) < PARALLEL_MIN_BYTES
    if small and not always:
        return None
    if small:
        common, kernels, jobs = "", [source], 1
    # longest first into the emptiest bin: compile time goes with the amount of kernel text
    bins: List[List[int]] = [[] for _ in range(min(jobs, len(kernels)))]
    load = [0] * len(bins)
    for i in sorted(range(len(kernels)), key=lambda i: -len(kernels[i])):
        b = load.index(min(load))
        bins[b].append(i)
        load[b] += len(kernels[i])
    load_library()  # built before the children look for it
    # Children that are to compile with the compiler of this process load its HIP libraries first: under torch
    # those are the ones the torch wheel carries (loaded before the C library, which then binds to them), and they
    # differ from the system's in version and in the code they generate.
    env = dict(os.environ)
    env.pop("OEQ_AMD_WORKER_PRELOAD", None)
    if own_compiler:
        env["OEQ_AMD_WORKER_PRELOAD"] = os.pathsep.join(_loaded_rocm_libraries().values())
    try:
        with tempfile.TemporaryDirectory(prefix="oeq_compile_") as tmp:
            procs = []
            for n, mine in enumerate(b for b in bins if b):
                src, out = Path(tmp) / f"part{n}.hip", Path(tmp) / f"part{n}.hsaco"
                src.write_text(common + "\n" + "\n".join(kernels[i] for i in sorted(mine)) + "\n")
                procs.append((out, subprocess.Popen(
                    [sys.executable, str(_WORKER_PATH), str(lib_path()), arch, str(src), str(out), *opts],
                    stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, env=env)))
            status = [proc.wait() for _out, proc in procs]  # (every child is waited for)
            for (out, _proc), rc in zip(procs, status):
                if rc == 3:  # the source does not compile: the compiler's log, as the in-process compile reports it
                    raise OeqError("oeq_jit_compile failed: " + Path(str(out) + ".err").read_text(errors="replace"))
            if any(status):
                return None
            blobs = [out.read_bytes() for out, _proc in procs]
            return blobs[0] if len(blobs) == 1 else pack_code(blobs)
    except OSError:
        return None


def _rocm_version(hip_library_file: str) -> Optional[Tuple[int, int, int]]:
    """(major, minor, patch) of a HIP runtime library, which ships with the hiprtc of the same release
    (hiprtcVersion names the API level, the same for both). Needs no GPU."""
    try:
        v = ctypes.c_int()
        if ctypes.CDLL(hip_library_file).hipRuntimeGetVersion(ctypes.byref(v)) != 0:
            return None
        return v.value // 10000000, v.value // 100000 % 100, v.value % 100000
    except (OSError, AttributeError):
        return None


_compiler_choice: Optional[Tuple[str, str]] = None


def compiler() -> Tuple[str, str]:
    """("process" | "system", release) of the hiprtc that kernels are compiled with. Inside a torch process the C
    library binds to the hiprtc of the torch wheel; a child process without torch gets the system's, which a
    torch-free caller of the C ABI also gets. ``OEQ_AMD_COMPILER=system`` has every kernel set compiled by child
    processes with that one (so that both kinds of caller run the same code objects); the default is the compiler of
    this process. The two releases at hand (ROCm 7.0 in the torch wheel, 7.2 in /opt/rocm) generate different code
    for nearly every kernel and the same speed: config 5's step 18.49 / 18.50 ms, forward 4.61 / 4.61 ms, in one run
    on one GPU. The release is part of a code object's name in the cache."""
    global _compiler_choice
    if _compiler_choice is None:
        import sys
        load_library()
        here = _rocm_version(_loaded_rocm_libraries().get("libamdhip64", "libamdhip64.so")) or (0, 0, 0)
        want = os.environ.get("OEQ_AMD_COMPILER", "")
        system = None
        if want == "system":
            # What a child process would compile with is asked of one, once: the answer is kept beside the code
            # objects, under the identity of the C library and of the system's ROCm directory, so that later
            # processes (one under a profiler, say) start no child for it.
            import json
            rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
            ident = hashlib.sha256(lib_path().read_bytes() + os.path.realpath(rocm).encode()).hexdigest()[:24]
            note = cache_dir() / "system_compiler.json"
            try:
                kept = json.loads(note.read_text())
                if kept.get("identity") == ident:
                    system = tuple(int(v) for v in kept["version"].split("."))
            except (OSError, ValueError, KeyError, AttributeError):
                system = None
            if system is None:
                try:
                    env = {k: v for k, v in os.environ.items() if k != "OEQ_AMD_WORKER_PRELOAD"}
                    res = subprocess.run([sys.executable, str(_WORKER_PATH), str(lib_path()), "--version"], env=env,
                                         capture_output=True, text=True, timeout=120)
                    if res.returncode == 0:
                        system = tuple(int(v) for v in res.stdout.split()[-1].split("."))
                        tmp = note.with_suffix(f".tmp{os.getpid()}")
                        tmp.write_text(json.dumps({"identity": ident, "version": "%d.%d.%d" % system}))
                        os.replace(tmp, note)
                except (OSError, ValueError, IndexError, subprocess.SubprocessError):
                    system = None
        if system is not None:
            _compiler_choice = ("system", "%d.%d.%d" % system)
        else:
            _compiler_choice = ("process", "%d.%d.%d" % here)
    return _compiler_choice


def cache_key(source: str, arch: str = DEFAULT_ARCH, options: Optional[Sequence[str]] = None) -> str:
    """Name of a kernel set's code object in the cache: the hash of what it is compiled from and the version of
    the compiler."""
    return f"{source_hash(source, arch, options)}-{compiler()[1]}"


def cache_path(source: str, arch: str = DEFAULT_ARCH, options: Optional[Sequence[str]] = None) -> Path:
    return cache_dir() / f"{cache_key(source, arch, options)}.hsaco"


def compile_source(source: str, arch: str = DEFAULT_ARCH, options: Optional[Sequence[str]] = None,
                   use_disk_cache: bool = True) -> bytes:
    """HIP source -> code object bytes, or a pack of them (hiprtc; needs no GPU)."""
    global _compiler_choice
    opts = list(options if options is not None else HIPRTC_OPTIONS)
    path = cache_path(source, arch, opts)
    if use_disk_cache and path.exists():
        return path.read_bytes()
    jobs = compile_jobs()
    blob = None
    if compiler()[0] == "system":
        blob = _compile_parallel(source, arch, opts, jobs, own_compiler=False, always=True)
        if blob is None:
            # no child could do it (or the source does not compile): from here on this process compiles itself,
            # and says so in the names of its code objects
            _compiler_choice = None
            os.environ["OEQ_AMD_COMPILER"] = "process"
            path = cache_path(source, arch, opts)
            if use_disk_cache and path.exists():
                return path.read_bytes()
    if blob is None and jobs > 1:
        blob = _compile_parallel(source, arch, opts, jobs)
    if blob is None:
        blob = _compile_one(source, arch, opts)
    if use_disk_cache:
        tmp = path.with_suffix(f".tmp{os.getpid()}")
        tmp.write_bytes(blob)
        os.replace(tmp, path)
    return blob


class KernelSet:
    """A loaded code object with its launch descriptors (oeq_kernels*)."""

    def __init__(self, code: bytes, dims: dict, descs: List[Tuple[int, str, int, int, int]]):
        lib = load_library()
        self._lib = lib
        self._names = [d[1].encode() for d in descs]
        arr = (_KernelDesc * len(descs))()
        for slot, desc, enc in zip(arr, descs, self._names):
            role, _name, block, upb, maxb = desc[:5]
            slot.role, slot.kernel_name, slot.block_threads = role, enc, block
            slot.units_per_block, slot.max_blocks = upb, maxb
            slot.grid_multiple = desc[5] if len(desc) > 5 else 0
        pd = _ProblemDims(**dims)
        handle = _P()
        _check(lib.oeq_kernels_create(code, len(code), ctypes.byref(pd), arr, len(descs), ctypes.byref(handle)),
               "oeq_kernels_create")
        self.handle = handle
        self.dims = dict(dims)

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                self._lib.oeq_kernels_destroy(self.handle)
                self.handle = None
        except Exception:
            pass

    def timing_enable(self, on: bool):
        _check(self._lib.oeq_kernel_timing_enable(self.handle, int(on)), "oeq_kernel_timing_enable")

    def timing_collect(self, role: int) -> Tuple[float, int]:
        """(summed milliseconds, launches) of the kernels of `role` recorded since the last call."""
        ms, n = ctypes.c_double(), _I64()
        _check(self._lib.oeq_kernel_timing_collect(self.handle, role, ctypes.byref(ms), ctypes.byref(n)),
               "oeq_kernel_timing_collect")
        return ms.value, n.value

    # thin wrappers; pointers are ints (tensor.data_ptr()), stream is an int
    def tp_forward(self, n, x, y, w, out, stream):
        _check(self._lib.oeq_tp_forward(self.handle, n, x, y, w, out, stream), "oeq_tp_forward")

    def tp_backward_workspace_bytes(self, n) -> int:
        return self._lib.oeq_tp_backward_workspace_bytes(self.handle, n)

    def tp_backward(self, n, x, dx, y, dy, w, dw, g, ws, ws_bytes, stream):
        _check(self._lib.oeq_tp_backward(self.handle, n, x, dx, y, dy, w, dw, g, ws, ws_bytes, stream),
               "oeq_tp_backward")

    def segment_sum_workspace_bytes(self, n_segments) -> int:
        return self._lib.oeq_segment_sum_workspace_bytes(self.handle, n_segments)

    def segment_sum(self, n_segments, n_items, row_len, src, dst, keys, perm, ws, ws_bytes, stream):
        _check(self._lib.oeq_segment_sum(self.handle, n_segments, n_items, row_len, src, dst, keys, perm, ws,
                                         ws_bytes, stream), "oeq_segment_sum")

    def grouped_sum_workspace_bytes(self, n_segments, n_items) -> int:
        return self._lib.oeq_grouped_sum_workspace_bytes(self.handle, n_segments, n_items)

    def grouped_sum(self, n_segments, n_items, row_len, src, dst, keys, ws, ws_bytes, stream):
        _check(self._lib.oeq_grouped_sum(self.handle, n_segments, n_items, row_len, src, dst, keys, ws, ws_bytes,
                                         stream), "oeq_grouped_sum")

    def conv_forward_workspace_bytes(self, nodes, nnz) -> int:
        return self._lib.oeq_conv_forward_workspace_bytes(self.handle, nodes, nnz)

    def conv_backward_workspace_bytes(self, nodes, nnz) -> int:
        return self._lib.oeq_conv_backward_workspace_bytes(self.handle, nodes, nnz)

    def conv_double_backward_workspace_bytes(self, nodes, nnz) -> int:
        return self._lib.oeq_conv_double_backward_workspace_bytes(self.handle, nodes, nnz)

    def conv_forward(self, nodes, nnz, x, y, w, out, rows, cols, ws, ws_bytes, stream):
        _check(self._lib.oeq_conv_forward(self.handle, nodes, nnz, x, y, w, out, rows, cols, ws, ws_bytes, stream),
               "oeq_conv_forward")

    def conv_forward_static(self, nodes, nnz, x, y, w, out, rows, cols, stream):
        """oeq_conv_forward with the library's static scratch array instead of a workspace; allocates nothing."""
        _check(self._lib.oeq_conv_forward_static(self.handle, nodes, nnz, x, y, w, out, rows, cols, stream),
               "oeq_conv_forward_static")

    # ---- index of an edge list, built once and shared by several calls
    def conv_index_bytes(self, nodes, nnz, sender_side: bool) -> int:
        return self._lib.oeq_conv_index_bytes(self.handle, nodes, nnz, int(sender_side))

    def conv_index_build(self, nodes, nnz, rows, cols, perm, sender_side: bool, index, index_bytes, stream):
        _check(self._lib.oeq_conv_index_build(self.handle, nodes, nnz, rows, cols, perm, int(sender_side), index,
                                              index_bytes, stream), "oeq_conv_index_build")

    INDEX_PIECES = ("rowptr", "colptr", "rperm", "sperm", "order", "hubptr", "hubnode", "shubptr", "shubnode")

    def conv_index_piece(self, nodes, nnz, sender_side: bool, piece: str) -> Tuple[int, int]:
        """(byte offset, int64 entries) of a piece of a built index (oeq_index_piece)."""
        off, n = _SZ(), _SZ()
        _check(self._lib.oeq_conv_index_piece(self.handle, nodes, nnz, int(sender_side),
                                              self.INDEX_PIECES.index(piece), ctypes.byref(off), ctypes.byref(n)),
               "oeq_conv_index_piece")
        return off.value, n.value

    def conv_forward_scratch_bytes(self, nodes, nnz) -> int:
        return self._lib.oeq_conv_forward_scratch_bytes(self.handle, nodes, nnz)

    def conv_forward_indexed(self, nodes, nnz, x, y, w, out, rows, cols, index, index_bytes, sender_side, scratch,
                             scratch_bytes, stream):
        _check(self._lib.oeq_conv_forward_indexed(self.handle, nodes, nnz, x, y, w, out, rows, cols, index, index_bytes,
                                                  int(sender_side), scratch, scratch_bytes, stream),
               "oeq_conv_forward_indexed")

    def conv_backward_scratch_bytes(self, nodes, nnz) -> int:
        return self._lib.oeq_conv_backward_scratch_bytes(self.handle, nodes, nnz)

    def conv_backward_indexed(self, nodes, nnz, x, dx, y, dy, w, dw, g, rows, cols, perm, index, index_bytes,
                              sender_side, scratch, scratch_bytes, stream):
        _check(self._lib.oeq_conv_backward_indexed(self.handle, nodes, nnz, x, dx, y, dy, w, dw, g, rows, cols, perm,
                                                   index, index_bytes, int(sender_side), scratch, scratch_bytes,
                                                   stream), "oeq_conv_backward_indexed")

    def conv_double_backward_scratch_bytes(self, nodes, nnz) -> int:
        return self._lib.oeq_conv_double_backward_scratch_bytes(self.handle, nodes, nnz)

    def conv_double_backward_indexed(self, nodes, nnz, x, y, w, g, ddx, ddy, ddw, dx, dy, dw, gg, rows, cols, perm,
                                     index, index_bytes, scratch, scratch_bytes, stream):
        _check(self._lib.oeq_conv_double_backward_indexed(self.handle, nodes, nnz, x, y, w, g, ddx, ddy, ddw, dx, dy, dw,
                                                          gg, rows, cols, perm, index, index_bytes, scratch,
                                                          scratch_bytes, stream), "oeq_conv_double_backward_indexed")

    def has_double_backward(self) -> bool:
        return bool(self._lib.oeq_has_double_backward(self.handle))

    def tp_double_backward_workspace_bytes(self, n) -> int:
        return self._lib.oeq_tp_double_backward_workspace_bytes(self.handle, n)

    def tp_double_backward(self, n, x, y, w, g, ddx, ddy, ddw, dx, dy, dw, gg, ws, ws_bytes, stream):
        _check(self._lib.oeq_tp_double_backward(self.handle, n, x, y, w, g, ddx, ddy, ddw, dx, dy, dw, gg, ws,
                                                ws_bytes, stream), "oeq_tp_double_backward")

    def conv_double_backward(self, nodes, nnz, x, y, w, g, ddx, ddy, ddw, dx, dy, dw, gg, rows, cols, perm, ws,
                             ws_bytes, stream):
        _check(self._lib.oeq_conv_double_backward(self.handle, nodes, nnz, x, y, w, g, ddx, ddy, ddw, dx, dy, dw, gg,
                                                  rows, cols, perm, ws, ws_bytes, stream), "oeq_conv_double_backward")

    def conv_backward(self, nodes, nnz, x, dx, y, dy, w, dw, g, rows, cols, perm, ws, ws_bytes, stream):
        _check(self._lib.oeq_conv_backward(self.handle, nodes, nnz, x, dx, y, dy, w, dw, g, rows, cols, perm, ws,
                                           ws_bytes, stream), "oeq_conv_backward")


_kernel_cache: Dict[str, KernelSet] = {}
_kernel_cache_lock = threading.Lock()


def get_kernel_set(source: str, dims: dict, descs: List[Tuple[int, str, int, int, int]],
                   arch: str = DEFAULT_ARCH) -> KernelSet:
    """Process-wide cache keyed by the source hash; compile happens under the lock
    (as in the reference, torch_core.hpp:192-231), launches do not."""
    key = source_hash(source, arch) + repr(sorted(dims.items())) + repr(descs)
    with _kernel_cache_lock:
        ks = _kernel_cache.get(key)
        if ks is None:
            ks = KernelSet(compile_source(source, arch), dims, descs)
            _kernel_cache[key] = ks
        return ks
