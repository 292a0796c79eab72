"""The C-ABI library loads, exports every symbol the header declares, compiles
generated sources for gfx950 with no GPU present and reports errors through
return codes. No kernel is launched here."""

import os
import re

import numpy as np
import pytest

from openequivariance_amd import runtime as rt
from openequivariance_amd.codegen.lower import lower
from openequivariance_amd.core import problems as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "oeq_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(oeq_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = rt.load_library()
    names = _declared_functions()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/oeq_amd.h but not exported"
    assert set(names) == set(rt.EXPORTS), "ctypes table and header disagree"
    assert lib.oeq_abi_version() == rt.ABI_VERSION


def test_compile_error_is_reported_not_fatal():
    with pytest.raises(rt.OeqError, match="hiprtc compile failed"):
        rt.compile_source("this is not HIP", use_disk_cache=False)
    blob = rt.compile_source('extern "C" __global__ void k(float* p) { p[threadIdx.x] = 1.0f; }', use_disk_cache=False)
    assert blob[:4] == b"\x7fELF"


def test_kernels_create_validates_arguments():
    lib = rt.load_library()
    dims = dict(L1_dim=4, L2_dim=1, L3_dim=4, weight_numel=1, elem_size=3, shared_weights=0, deterministic=0,
                wpartial_per_block=0)
    with pytest.raises(rt.OeqError, match="elem_size"):
        rt.KernelSet(b"\x7fELFxxxx", dims, [(rt.ROLE_TP_FORWARD, "forward", 64, 1, 0)])
    dims["elem_size"] = 4
    with pytest.raises(rt.OeqError, match="descriptor"):
        rt.KernelSet(b"\x7fELFxxxx", dims, [(rt.ROLE_TP_FORWARD, "forward", 0, 1, 0)])
    ks = rt.KernelSet(b"\x7fELFxxxx", dims, [(rt.ROLE_TP_FORWARD, "forward", 64, 1, 0)])
    # zero-sized work returns before touching the device; bad sizes are rejected
    assert lib.oeq_tp_forward(ks.handle, 0, None, None, None, None, None) == 0
    assert lib.oeq_tp_forward(ks.handle, -1, None, None, None, None, None) == -1
    assert b"negative" in lib.oeq_last_error()
    assert lib.oeq_tp_forward(None, 1, None, None, None, None, None) == -1
    assert ks.conv_forward_workspace_bytes(10, 10) == 0
    dims["deterministic"] = 1
    ks2 = rt.KernelSet(b"\x7fELFxxxx", dims, [(rt.ROLE_CONV_FORWARD, "forward", 64, 1, 0)])
    # segment starts: 31 + 1 entries, one count and a list of 126 long segments, 8 bytes each -> 1272 -> 1280
    assert ks2.conv_forward_workspace_bytes(31, 10) == 1280
    assert ks2.conv_backward_workspace_bytes(31, 10) == 2 * 1280 + 256  # 10*4*4 = 160 -> 256


ALL = [P.config1_single_uvu, P.config2_nequip_uvu, P.config3_mace_uvu, P.config4_uvw_shared,
       lambda: P.config3_mace_uvu(np.float64)]


@pytest.mark.parametrize("make", ALL)
def test_generated_tp_sources_compile_for_gfx950(make):
    from openequivariance_amd._torch.tensor_product import build_tp_module
    src, dims, descs = build_tp_module(make())
    blob = rt.compile_source(src)
    assert all(part[:4] == b"\x7fELF" for part in rt.unpack_code(blob))
    names = {d[1] for d in descs}
    assert {"forward", "backward"} <= names
    for n in names:
        assert n.encode() in blob


@pytest.mark.parametrize("det", [False, True])
@pytest.mark.parametrize("make", [P.config1_single_uvu, P.config2_nequip_uvu, P.config5_mace_conv,
                                  lambda: P.config5_mace_conv(np.float64)])
def test_generated_conv_sources_compile_for_gfx950(make, det):
    from openequivariance_amd._torch.tensor_product_conv import build_conv_module
    src, dims, descs = build_conv_module(make(), det)
    blob = rt.compile_source(src)
    names = {d[1] for d in descs}
    assert {"forward", "backward", "fixup_backward"} <= names
    # the counting-sort kernels serve the edge grouping (deterministic=False) and, in both modes, the walk order
    assert {"oeq_group_count", "oeq_group_scan", "oeq_group_scatter", "oeq_group_order", "oeq_order_hop"} <= names
    assert dims["deterministic"] == (rt.CONV_SORTED if det else rt.CONV_GROUPED)
    # generated code must not carry packed-FP32 arithmetic or anything CUDA-flavoured
    assert "__syncwarp" not in src and "cuda" not in src.lower()


def test_float_atomics_conv_kernels_compile(monkeypatch):
    from openequivariance_amd._torch.tensor_product_conv import build_conv_module
    monkeypatch.setenv("OEQ_AMD_TUNE", "conv_sort=0")
    src, dims, descs = build_conv_module(P.config5_mace_conv(), False)
    assert dims["deterministic"] == rt.CONV_ATOMIC and "fixup_backward" not in {d[1] for d in descs}
    assert "oeq_atomic_add" in src and len(rt.compile_source(src)) > 0


def _elf_functions(blob: bytes):
    """{name: machine code} of the function symbols an ELF64 code object defines."""
    import struct
    shoff, = struct.unpack_from("<Q", blob, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", blob, 0x3A)
    sections = [struct.unpack_from("<IIQQQQIIQQ", blob, shoff + i * shentsize) for i in range(shnum)]
    out = {}
    for _name, kind, _flags, _addr, off, size, link, _info, _align, entsize in sections:
        if kind != 2:  # SHT_SYMTAB
            continue
        str_off = sections[link][4]
        for at in range(off, off + size, entsize):
            st_name, st_info, _other, st_shndx, st_value, st_size = struct.unpack_from("<IBBHQQ", blob, at)
            if st_info & 0xF == 2 and 0 < st_shndx < shnum:  # STT_FUNC, defined
                end = blob.index(b"\0", str_off + st_name)
                sec = sections[st_shndx]
                start = sec[4] + st_value - sec[3]
                out[blob[str_off + st_name:end].decode()] = blob[start:start + st_size]
    return out


def test_large_kernel_sets_compile_side_by_side(monkeypatch, tmp_path):
    """A module above the size limit is split at its kernel definitions, the shares are compiled by child
    processes and come back as one pack that the library accepts; a kernel inside a namespace keeps it."""
    from openequivariance_amd._torch.tensor_product_conv import build_conv_module
    # (last layer: its sender gradients come from a kernel emitted inside a namespace of its own)
    src, dims, descs = build_conv_module(P.nequix_problems()[2], True)
    assert "namespace oeq_dx {" in src
    common, kernels = rt.split_kernels(src)
    assert "__global__" not in common and len(kernels) == src.count('extern "C" __global__')
    inside = [k for k in kernels if k.startswith("namespace oeq_dx {")]
    assert len(inside) == 1 and "void backward_dx(" in inside[0]
    names = {d[1] for d in descs}
    assert all(sum(f" {n}(" in k.split("\n")[1 if k.startswith("namespace") else 0] for k in kernels) == 1
               for n in names)
    monkeypatch.setattr(rt, "PARALLEL_MIN_BYTES", 0)
    monkeypatch.setenv("OEQ_AMD_COMPILE_JOBS", "3")
    monkeypatch.setenv("OEQ_AMD_CACHE_DIR", str(tmp_path))
    # with the compiler of this process (under torch: the hiprtc of the torch wheel)
    monkeypatch.setenv("OEQ_AMD_COMPILER", "process")
    monkeypatch.setattr(rt, "_compiler_choice", None)
    assert rt.compiler()[0] == "process"
    blob = rt.compile_source(src)
    parts = rt.unpack_code(blob)
    assert blob.startswith(rt.PACK_MAGIC) and len(parts) == 3 and all(p[:4] == b"\x7fELF" for p in parts)
    assert rt.pack_code(parts) == blob and rt.cache_path(src).read_bytes() == blob
    assert rt.cache_path(src).name == f"{rt.source_hash(src)}-{rt.compiler()[1]}.hsaco"
    defined = [_elf_functions(p) for p in parts]
    for n in names:  # every kernel in exactly one code object
        assert sum(n in d for d in defined) == 1, n
    rt.KernelSet(blob, dims, descs)
    # one job: compiled in this process
    monkeypatch.setenv("OEQ_AMD_COMPILE_JOBS", "1")
    whole = rt.compile_source(src, use_disk_cache=False)
    assert whole[:4] == b"\x7fELF"
    # The children loaded this process's HIP libraries first and so compiled with the same hiprtc (the system's
    # generates other code): kernels that make no reference to other symbols are the same bytes.
    code = _elf_functions(whole)
    for part in defined:
        for name in ("oeq_hub_fill", "oeq_segment_sum"):
            if name in part:
                assert part[name] == code[name], name
        assert all(len(part[name]) == len(code[name]) for name in part if name in names)
    # a child that cannot be run: compiled in this process
    monkeypatch.setenv("OEQ_AMD_COMPILE_JOBS", "3")
    worker = rt._WORKER_PATH
    monkeypatch.setattr(rt, "_WORKER_PATH", tmp_path / "missing.py")
    assert rt.compile_source(src, use_disk_cache=False) == whole
    monkeypatch.setattr(rt, "_WORKER_PATH", worker)
    # with the system's hiprtc: every compile runs in a child process, the code object is named for that release;
    # when no child can be run the process goes back to its own compiler
    monkeypatch.setenv("OEQ_AMD_COMPILER", "system")
    monkeypatch.setattr(rt, "_compiler_choice", None)
    if rt.compiler()[0] == "system":
        other = rt.compile_source(src)
        assert rt.cache_path(src).read_bytes() == other and rt.compiler()[1] in rt.cache_path(src).name
        monkeypatch.setenv("OEQ_AMD_COMPILE_JOBS", "1")
        one = rt.compile_source(src, use_disk_cache=False)
        assert one[:4] == b"\x7fELF" and {k: len(v) for k, v in _elf_functions(one).items()} == \
            {k: len(v) for p in rt.unpack_code(other) for k, v in _elf_functions(p).items()}
        monkeypatch.setattr(rt, "_WORKER_PATH", tmp_path / "missing.py")
        assert rt.compile_source(src, use_disk_cache=False) == whole and rt.compiler()[0] == "process"
    monkeypatch.setattr(rt, "_compiler_choice", None)


def test_forward_kernel_that_spills_gives_way_to_one_wave_per_node():
    """Waves that share a node's output segments: where the compiler cannot fit that kernel into its registers (the
    code object's kernel descriptor shows scratch memory), the module is generated again with one wave per node."""
    from openequivariance_amd._torch.tensor_product_conv import build_conv_module
    harmonics = "1x0e+1x1e+1x2e+1x3e"
    problem = P.CTPP("64x0e+64x1e+64x2e+64x3e", harmonics, "0e+1e+2e+3e", "four-irreps-even")
    os.environ.pop("OEQ_AMD_TUNE", None)
    src, _dims, descs = build_conv_module(problem, True)
    forward = next(d for d in descs if d[1] == "forward")
    assert forward[2] == 64 and forward[3] == 1                     # one wave, one node per block
    assert rt.kernel_resources(rt.compile_source(src))["forward"][1] == 0
    # the shared form, forced: three waves per node, and it spills
    os.environ["OEQ_AMD_TUNE"] = "conv_segw=4"
    try:
        src, _dims, descs = build_conv_module(problem, True)
    finally:
        os.environ.pop("OEQ_AMD_TUNE", None)
    forward = next(d for d in descs if d[1] == "forward")
    assert forward[2] == 192 and rt.kernel_resources(rt.compile_source(src))["forward"][1] > 64
    # a problem whose shared form fits keeps it (mixed multiplicities, three segments)
    src, _dims, descs = build_conv_module(P.seven_net_problems()[1], True)
    forward = next(d for d in descs if d[1] == "forward")
    assert forward[2] == 192 and forward[3] == 1 and rt.kernel_resources(rt.compile_source(src))["forward"][1] == 0


def test_forward_kernel_takes_a_third_wave_where_that_costs_no_scratch_memory():
    """A forward kernel that the compiler gave more than a third of a SIMD's registers is generated again held
    to a third, and that form is kept where its code object shows no scratch memory."""
    from openequivariance_amd._torch.tensor_product_conv import build_conv_module

    def forward_bounds(src):
        head = src[:src.index("void forward(")]
        return re.findall(r"amdgpu_waves_per_eu\(([^)]*)\)", head)[-1].replace(" ", "")

    os.environ.pop("OEQ_AMD_TUNE", None)
    harmonics = "1x0e+1x1o+1x2e+1x3o"
    fits = P.CTPP("96x0e+96x1o+96x2e+96x3o", harmonics, "0e+1o+2e+3o", "96-channels")
    src, _dims, _descs = build_conv_module(fits, True)
    assert forward_bounds(src) == "3,3"
    blob = rt.compile_source(src)
    assert rt.kernel_registers(blob)["forward"] <= 168 and rt.kernel_resources(blob)["forward"][1] == 0
    os.environ["OEQ_AMD_TUNE"] = "conv_wf=23"
    try:
        src, _dims, _descs = build_conv_module(fits, True)
    finally:
        os.environ.pop("OEQ_AMD_TUNE", None)
    assert forward_bounds(src) == "2,3" and rt.kernel_registers(rt.compile_source(src))["forward"] > 168
    # held to a third this kernel would spill: it keeps its two waves
    spills = P.CTPP("128x0e+96x1e+64x2e", harmonics.replace("o", "e"), "0e+1e+2e", "mixed-channels")
    src, _dims, _descs = build_conv_module(spills, True)
    assert forward_bounds(src) == "2,3" and rt.kernel_registers(rt.compile_source(src))["forward"] > 168
    # double precision keeps the plain budget of two waves
    src, _dims, _descs = build_conv_module(P.CTPP("96x0e+96x1o+96x2e+96x3o", harmonics, "0e+1o+2e+3o", "96-channels-f64",
                                                  irrep_dtype=np.float64, weight_dtype=np.float64), True)
    assert forward_bounds(src) == "2,2"


def test_malformed_code_packs_are_rejected():
    import struct
    dims = dict(L1_dim=4, L2_dim=4, L3_dim=4, weight_numel=4, elem_size=4)
    desc = [(rt.ROLE_TP_FORWARD, "forward", 64, 1, 0)]
    elf = b"\x7fELF" + b"x" * 60
    rt.KernelSet(rt.pack_code([elf, elf]), dims, desc)
    for bad in (rt.PACK_MAGIC + struct.pack("<Q", 0),                          # no code object
                rt.PACK_MAGIC + struct.pack("<QQ", 2, 64) + b"\0" * 200,        # count beyond the sizes present
                rt.PACK_MAGIC + struct.pack("<QQ", 1, 1 << 40) + b"\0" * 200,   # size beyond the pack
                rt.PACK_MAGIC + struct.pack("<QQ", 1, 0) + b"\0" * 200,         # empty code object
                rt.pack_code([elf, elf])[:-1]):                                 # truncated
        with pytest.raises(rt.OeqError, match="malformed code pack"):
            rt.KernelSet(bad, dims, desc)


def test_lowering_lane_mapping():
    low = lower(P.config3_mace_uvu())
    assert (low.lanes_per_row, low.rows_per_wave, low.n_chunks) == (64, 1, 2)
    low = lower(P.config2_nequip_uvu())
    assert (low.lanes_per_row, low.rows_per_wave, low.n_chunks) == (32, 2, 1)
    low = lower(P.config1_single_uvu())
    assert (low.lanes_per_row, low.rows_per_wave, low.n_chunks) == (1, 64, 1)
    assert lower(P.config3_mace_uvu()).flops("forward") == 148224
    assert lower(P.config3_mace_uvu()).flops("backward") == 406656
    assert lower(P.config2_nequip_uvu()).flops("forward") == 13376
