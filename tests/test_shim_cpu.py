"""The interception shim without a GPU: its code-object reader against an independent decoder
and against the C argument-passing rules, malformed input, and the library's exports.

The checker (this file) decodes the same files with Python's `msgpack` and `struct` modules;
the expected layouts of three kernels are also written out by hand from their C signatures
(natural alignment of each argument in the kernel argument segment)."""
import ctypes
import os
import random
import re
import struct
import subprocess

import msgpack
import pytest

import xsched_amd as xs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "xsched_amd", "lib")
BUNDLE_MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


def _elf_metadata(elf):
    """{kernel name: [(offset, size), ...]} of the explicit arguments, decoded independently."""
    phoff = struct.unpack_from("<Q", elf, 0x20)[0]
    phentsize, phnum = struct.unpack_from("<HH", elf, 0x36)
    for k in range(phnum):
        p_type, _, p_offset, _, _, p_filesz = struct.unpack_from("<IIQQQQ", elf, phoff + k * phentsize)
        if p_type != 4:
            continue
        q = p_offset
        while q < p_offset + p_filesz:
            namesz, descsz, ntype = struct.unpack_from("<III", elf, q)
            q += 12
            name = elf[q:q + namesz]
            q += (namesz + 3) & ~3
            desc = elf[q:q + descsz]
            q += (descsz + 3) & ~3
            if name.rstrip(b"\0") == b"AMDGPU" and ntype == 32:
                md = msgpack.unpackb(desc, raw=False)
                return {kern[".name"]: [(a[".offset"], a[".size"]) for a in kern.get(".args", [])
                                        if not a.get(".value_kind", "").startswith("hidden_")]
                        for kern in md["amdhsa.kernels"]}
    raise AssertionError("no AMDGPU metadata note")


def _bundle_of(path):
    data = open(path, "rb").read()
    at = data.find(BUNDLE_MAGIC)
    assert at >= 0, path
    n = struct.unpack_from("<Q", data, at + 24)[0]
    p = at + 32
    end = 0
    device = None
    for _ in range(n):
        off, size, tl = struct.unpack_from("<QQQ", data, p)
        triple = data[p + 24:p + 24 + tl]
        p += 24 + tl
        end = max(end, off + size)
        if b"amdgcn" in triple and size:
            device = data[at + off:at + off + size]
    return data[at:at + end], device


def _layout(image, kernel, size=None, cap=64):
    lib = xs.shimhip()
    buf = ctypes.create_string_buffer(bytes(image), len(image))
    offsets = (ctypes.c_uint32 * cap)()
    sizes = (ctypes.c_uint32 * cap)()
    n = ctypes.c_size_t(0)
    res = lib.HipShimKernelArgLayout(ctypes.cast(buf, ctypes.c_void_p), len(image) if size is None else size,
                                     kernel.encode(), offsets, sizes, cap, ctypes.byref(n))
    return res, [(offsets[i], sizes[i]) for i in range(min(n.value, cap))], n.value


@pytest.fixture(scope="module")
def app_bundle():
    path = os.path.join(LIB, "shim_app_plain")
    assert os.path.exists(path), "run python -m xsched_amd.build"
    return _bundle_of(path)


def test_library_exports_what_its_header_declares():
    out = subprocess.run(["nm", "-D", "--defined-only", os.path.join(LIB, "libshimhip.so")],
                         capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    header = open(os.path.join(ROOT, "include", "xsched", "hip", "shim.h")).read()
    declared = re.findall(r"^XResult\s+(\w+)\s*\(", header, flags=re.M)
    assert set(declared) == set(xs.SHIMHIP_API) and len(declared) == 2
    for name in declared:
        assert name in exported
    # every HIP entry point the header lists as intercepted is defined by the library
    listed = set(re.findall(r"\b(__hip\w+|hip[A-Z]\w+)", header.split("Intercepted:")[1].split("The two functions")[0]))
    assert len(listed) >= 45
    assert listed <= exported, sorted(listed - exported)
    hip_defined = {n for n in exported if n.startswith("hip") or n.startswith("__hip")}
    assert hip_defined == listed, sorted(hip_defined ^ listed)


def test_layouts_match_the_independent_decoder(app_bundle):
    bundle, device = app_bundle
    want = _elf_metadata(device)
    assert len(want) >= 7
    for kernel, args in want.items():
        for image in (bundle, device):         # offload bundle and bare code object
            res, got, n = _layout(image, kernel)
            assert res == xs.kXSchedSuccess, kernel
            assert n == len(args) and got == args, kernel
    # the same with the size unknown, as for __hipRegisterFatBinary
    res, got, _ = _layout(bundle, next(iter(want)), size=0)
    assert res == xs.kXSchedSuccess and got == want[next(iter(want))]


def test_layouts_follow_the_c_signatures(app_bundle):
    bundle, _ = app_bundle
    by_hand = {
        # float a, const float *x, float *y, size_t n
        "_Z5SaxpyfPKfPfm": [(0, 4), (8, 8), (16, 8), (24, 8)],
        # struct {float; double; char} (24 bytes), short, unsigned char, double *, int
        "_Z5Mixed4PairshPdi": [(0, 24), (24, 2), (26, 1), (32, 8), (40, 4)],
        # struct of 50 uint32_t by value, uint32_t *
        "_Z7SumWide4WidePj": [(0, 200), (200, 8)],
        "_Z4Bumpv": [],
        # float *, float, uint32_t, then the 40-byte XGuardArgs the shim recognises by this name
        "_Z13AffineGuardedPffj10XGuardArgs": [(0, 8), (8, 4), (12, 4), (16, 40)],
    }
    for kernel, args in by_hand.items():
        res, got, n = _layout(bundle, kernel)
        assert res == xs.kXSchedSuccess, kernel
        assert got == args and n == len(args), kernel


def test_module_code_object():
    path = os.path.join(LIB, "shim_module.co")
    image = open(path, "rb").read()
    device = _bundle_of(path)[1] if image.startswith(BUNDLE_MAGIC) else image
    want = _elf_metadata(device)
    assert want["ModScale"] == [(0, 8), (8, 4), (12, 4)]
    assert want["ModShift"] == [(0, 8), (8, 2), (12, 4)]
    for kernel, args in want.items():
        assert _layout(image, kernel)[:2] == (xs.kXSchedSuccess, args)


def _packed_bundle(path):
    """(compressed image as it sits in the file, the bundle it unpacks to) - unpacked here with
    pyarrow's zstd codec, the library under test uses the system's libzstd."""
    import pyarrow as pa
    data = open(path, "rb").read()
    at = data.find(b"CCOB")
    assert at >= 0
    version, method = struct.unpack_from("<HH", data, at + 4)
    assert (version, method) == (3, 1), "hipcc of this image writes version 3 headers with zstd"
    file_size, raw_size = struct.unpack_from("<QQ", data, at + 8)
    packed = data[at:at + file_size]
    raw = pa.Codec("zstd").decompress(packed[32:], decompressed_size=raw_size).to_pybytes()
    assert raw.startswith(BUNDLE_MAGIC)
    return packed, raw


def test_compressed_bundles(app_bundle):
    packed, raw = _packed_bundle(os.path.join(LIB, "shim_app_packed"))
    end, device = 0, None
    n = struct.unpack_from("<Q", raw, 24)[0]
    p = 32
    for _ in range(n):
        off, size, tl = struct.unpack_from("<QQQ", raw, p)
        if b"amdgcn" in raw[p + 24:p + 24 + tl] and size:
            device = raw[off:off + size]
        p += 24 + tl
    want = _elf_metadata(device)
    assert want == _elf_metadata(app_bundle[1])     # same program, same layouts
    for kernel, args in want.items():
        assert _layout(packed, kernel)[:2] == (xs.kXSchedSuccess, args)
        assert _layout(packed, kernel, size=0)[:2] == (xs.kXSchedSuccess, args)   # size from the header
    # the earlier header forms, built here around the same compressed bytes
    body, raw_size = packed[32:], len(raw)
    v2 = b"CCOB" + struct.pack("<HHII", 2, 1, 24 + len(body), raw_size) + packed[24:32] + body
    v1 = b"CCOB" + struct.pack("<HHI", 1, 1, raw_size) + packed[24:32] + body
    assert _layout(v2, "_Z5SaxpyfPKfPfm")[:2] == (xs.kXSchedSuccess, want["_Z5SaxpyfPKfPfm"])
    assert _layout(v1, "_Z5SaxpyfPKfPfm")[:2] == (xs.kXSchedSuccess, want["_Z5SaxpyfPKfPfm"])
    assert _layout(v1, "_Z5SaxpyfPKfPfm", size=0)[0] == xs.kXSchedErrorNotSupported   # version 1 has no length
    # zlib (method 0)
    import zlib
    z = zlib.compress(raw)
    v3z = b"CCOB" + struct.pack("<HHQQ", 3, 0, 32 + len(z), raw_size) + packed[24:32] + z
    assert _layout(v3z, "_Z5SaxpyfPKfPfm")[:2] == (xs.kXSchedSuccess, want["_Z5SaxpyfPKfPfm"])
    # damage: wrong sizes, cut data, unknown method or version
    bad_raw = bytearray(packed); struct.pack_into("<Q", bad_raw, 16, raw_size + 1)
    assert _layout(bytes(bad_raw), "_Z5SaxpyfPKfPfm")[0] == xs.kXSchedErrorNotSupported
    assert _layout(packed[:len(packed) // 2], "_Z5SaxpyfPKfPfm")[0] == xs.kXSchedErrorInvalidValue
    cut = bytearray(packed[:len(packed) - 40]); struct.pack_into("<Q", cut, 8, len(cut))
    assert _layout(bytes(cut), "_Z5SaxpyfPKfPfm")[0] == xs.kXSchedErrorNotSupported
    method9 = bytearray(packed); struct.pack_into("<H", method9, 6, 9)
    assert _layout(bytes(method9), "_Z5SaxpyfPKfPfm")[0] == xs.kXSchedErrorNotSupported
    version9 = bytearray(packed); struct.pack_into("<H", version9, 4, 9)
    assert _layout(bytes(version9), "_Z5SaxpyfPKfPfm")[0] == xs.kXSchedErrorNotSupported


def test_more_arguments_than_room(app_bundle):
    bundle, _ = app_bundle
    res, got, n = _layout(bundle, "_Z5Mixed4PairshPdi", cap=2)
    assert res == xs.kXSchedSuccess and n == 5 and got == [(0, 24), (24, 2)]
    lib = xs.shimhip()
    buf = ctypes.create_string_buffer(bytes(bundle), len(bundle))
    count = ctypes.c_size_t(0)
    assert lib.HipShimKernelArgLayout(ctypes.cast(buf, ctypes.c_void_p), len(bundle), b"_Z4Bumpv", None, None, 0,
                                      ctypes.byref(count)) == xs.kXSchedSuccess and count.value == 0
    assert lib.HipShimKernelArgLayout(ctypes.cast(buf, ctypes.c_void_p), len(bundle), b"_Z4Bumpv", None, None, 4,
                                      ctypes.byref(count)) == xs.kXSchedErrorInvalidValue
    assert lib.HipShimKernelArgLayout(None, 0, b"x", None, None, 0, ctypes.byref(count)) == xs.kXSchedErrorInvalidValue


def test_unknown_kernel_and_foreign_bytes(app_bundle):
    bundle, device = app_bundle
    assert _layout(bundle, "NoSuchKernel")[0] == xs.kXSchedErrorNotFound
    assert _layout(b"not a code object at all" * 4, "k")[0] == xs.kXSchedErrorInvalidValue
    assert _layout(b"CCOB" + b"\0" * 60, "k")[0] == xs.kXSchedErrorNotSupported     # compressed, version 0
    assert _layout(b"\x7fELF" + b"\x01\x01" + b"\0" * 58, "k")[0] == xs.kXSchedErrorInvalidValue  # 32-bit ELF
    host_only = BUNDLE_MAGIC + struct.pack("<QQQQ", 1, 64, 0, 4) + b"host"
    assert _layout(host_only + b"\0" * 32, "k")[0] == xs.kXSchedErrorInvalidValue    # no amdgcn entry


def test_truncated_images_are_refused_not_read_past(app_bundle):
    bundle, device = app_bundle
    kernel = "_Z5SaxpyfPKfPfm"
    for image in (bundle, device):
        cuts = sorted(set(list(range(0, 200, 7)) + list(range(200, len(image), 211)) + [len(image) - 1]))
        refused = 0
        for cut in cuts:
            res, got, _ = _layout(image[:cut] + b"\xee" * 16, kernel, size=cut)  # the tail must never be looked at
            if res == xs.kXSchedSuccess:
                # a bare code object cut behind its metadata note still holds all that is read
                assert image is device and got == [(0, 4), (8, 8), (16, 8), (24, 8)], cut
            else:
                assert res in (xs.kXSchedErrorInvalidValue, xs.kXSchedErrorNotFound), cut
                refused += 1
        assert refused >= 30


def test_corrupted_metadata_never_crashes(app_bundle):
    _, device = app_bundle
    want = _elf_metadata(device)
    rng = random.Random(11)
    outcomes = set()
    for _ in range(300):
        image = bytearray(device)
        for _ in range(rng.randint(1, 8)):
            image[rng.randrange(len(image))] = rng.randrange(256)
        res, got, _ = _layout(bytes(image), "_Z5SaxpyfPKfPfm")
        outcomes.add(res)
        if res == xs.kXSchedSuccess and image == bytearray(device):
            assert got == want["_Z5SaxpyfPKfPfm"]
    assert outcomes <= {xs.kXSchedSuccess, xs.kXSchedErrorInvalidValue, xs.kXSchedErrorNotFound}


def test_reader_under_address_and_ub_sanitizers(tmp_path):
    """The reader takes bytes it has not produced: built with -fsanitize=address,undefined it
    reads thousands of damaged and truncated copies of the three real images from heap blocks
    of exactly the stated size (tests/code_object_fuzz.cpp), and nothing must be flagged."""
    exe = str(tmp_path / "co_fuzz")
    shim = os.path.join(ROOT, "xsched_amd", "csrc", "shim")
    # the sanitizer runtimes are linked statically: they then do not mind other preloaded libraries
    subprocess.run(["g++", "-std=c++20", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                    "-static-libasan", "-static-libubsan",
                    "-I", shim, os.path.join(shim, "code_object.cpp"), os.path.join(ROOT, "tests", "code_object_fuzz.cpp"),
                    "-o", exe, "-ldl"], check=True, capture_output=True)
    images = [os.path.join(LIB, n) for n in ("shim_app_plain", "shim_app_packed", "shim_module.co")]
    proc = subprocess.run([exe, "1500"] + images, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-4000:]
    lines = proc.stdout.strip().splitlines()
    assert len(lines) == 3 and all("refused" in line for line in lines), proc.stdout
    assert lines[0].split(":")[1].strip().startswith("11 kernels") and lines[2].split(":")[1].strip().startswith("2 kernels")
