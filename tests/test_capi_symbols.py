"""CPU: the C-ABI library loads and exports every symbol include/wekua_hip.h declares; the
Python binding declares a signature for each; host-only entry points behave; and without a GPU
the product path fails loudly instead of falling back to anything."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "wekua_hip.h")
TEST_HEADER = os.path.join(ROOT, "include", "wekua_hip_test.h")     # knobs for tests, benchmarks and profiles
TEST_ONLY = {"wk_gemm_variant", "wk_gemm_variant_with_workspace", "wk_gemm_split_plan", "wk_gemm_force_variant",
             "wk_test_option", "wk_copy_kernel", "wk_probe_launch", "wk_stream_probe"}


def declared_functions(headers=(HEADER, TEST_HEADER)):
    names = set()
    for h in headers:
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names |= set(re.findall(r"\b(wk_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_test_knobs_are_not_in_the_product_header():
    """What exposes or overrides the library's own choices lives in wekua_hip_test.h, and the library reads
    no switch from the environment."""
    assert not TEST_ONLY & set(declared_functions((HEADER,)))
    assert set(declared_functions((TEST_HEADER,))) == TEST_ONLY
    csrc = os.path.join(ROOT, "wekua_amd", "csrc")
    for f in os.listdir(csrc):
        assert "getenv" not in open(os.path.join(csrc, f)).read(), f
    from wekua_amd import _capi
    lib = _capi.load()
    assert lib.wk_test_option(b"no-such-switch", 1) == 1
    for name, default in ((b"gemm_walk_rows", 0), (b"tail_strict", 0), (b"alloc_colours", 1), (b"stream_k", 1), (b"strips", 1), (b"persistent", 1), (b"skinny", 1)):
        assert lib.wk_test_option(name, default) == 0


def test_kernel_choice_by_name_without_a_device():
    """The name query runs the cost model on the host (256 compute units assumed): products whose tiles do not
    come out even over the units take the kernels that deal their left-over tiles by k-slabs, whole rounds do
    not, and the two switches of the test header take them, and the strips, away."""
    from wekua_amd import _capi, raw
    lib = _capi.load()

    def name(dtype, M, N, K):
        per = 4 if dtype == "f32" else 2
        up = lambda n: -(-n // per) * per
        return lib.wk_gemm_variant(raw.dtype_id(dtype), 0, 0, M, N, K, up(K), up(N), up(N), None, None, None).decode()
    assert name("f32", 2500, 2500, 2500) == "mfma_f32_128x128k"
    assert name("f32", 1536, 1536, 1536) == "mfma_f32_64x64k"
    assert name("f32", 4300, 4300, 4300) == "mfma_f32_256x128k"
    assert name("f64", 1536, 1536, 1536) == "mfma_f64_64x64k"
    assert name("f64", 3456, 3456, 3456) == "mfma_f64_128x128k"
    for whole_rounds in (("f32", 8192, 8192, 8192), ("f32", 4096, 4096, 4096), ("f32", 2048, 4096, 1024), ("f32", 1024, 1024, 1024),
                         ("f64", 4096, 4096, 4096), ("f64", 8192, 256, 8192)):
        assert not name(*whole_rounds).endswith("k"), whole_rounds
    assert name("f32", 1536, 1536, 192).endswith("d")                    # k below 256: the exchange would not pay
    assert name("f32", 1536, 1536, 384) == "mfma_f32_64x64k"              # (measured: 24 us plain, 21 dealt)
    assert name("f32", 4097, 4095, 4093) == "mfma_f32_256x128d+strips"   # one row beyond sixteen tiles: in parts
    assert name("f32", 2200, 2200, 2200) == "mfma_f32_64x64d"            # strips of 24: three more launches would cost more
    try:
        assert lib.wk_test_option(b"stream_k", 0) == 0
        assert not name("f32", 2500, 2500, 2500).endswith("k")
        assert not name("f64", 1536, 1536, 1536).endswith("k")
        assert lib.wk_test_option(b"strips", 0) == 0
        assert "+strips" not in name("f32", 4097, 4095, 4093)
    finally:
        lib.wk_test_option(b"stream_k", 1)
        lib.wk_test_option(b"strips", 1)


def test_header_declares_the_hot_path():
    names = declared_functions()
    for must in ("wk_gemm", "wk_axpy", "wk_device_open", "wk_stream_create", "wk_malloc", "wk_copy_h2d_rect_async",
                 "wk_copy_d2h_rect_async", "wk_fill", "wk_identity", "wk_stream_sync", "wk_strerror"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from wekua_amd import _capi
    lib = _capi.load()
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in the headers but not exported: {missing}"


def test_binding_covers_every_declared_symbol():
    from wekua_amd import _capi
    declared = set(declared_functions())
    bound = set(_capi.SIGNATURES)
    assert declared == bound, f"unbound: {declared - bound}; undeclared: {bound - declared}"


def test_k_split_plans_fit_the_scratch_and_the_counters():
    """Host arithmetic of the GEMM that splits k over work-groups: whatever the shape, a plan that
    splits covers k exactly with whole slabs per share, and its partial tiles and arrival counters
    fit what every stream owns (128 MiB, 4096 counters) -- the kernel takes both for granted."""
    from wekua_amd import _capi
    lib = _capi.load()
    u32, u64, sz = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_size_t
    seen_split = 0
    for dtype, es, name in ((8, 4, b"mfma_f32_64x64z"), (9, 8, b"mfma_f64_64x64z")):
        for forced in (None, name):
            for (M, N, K) in [(512, 512, 8192), (512, 512, 512), (64, 64, 100000), (300, 200, 2500), (70, 45, 97), (1, 1, 1),
                              (1, 1, 64), (64, 64, 33), (2048, 2048, 8192), (8192, 256, 8192), (4096, 4096, 65), (1024, 64, 4096),
                              (100000, 64, 4096), (64, 262144, 4096), (768, 768, 3000), (5000, 3000, 128)]:
                shares, klen, first, tiles, nbytes = u32(), u32(), u64(), u64(), sz()
                assert lib.wk_gemm_split_plan(dtype, 0, 1, M, N, K, forced, shares, klen, first, tiles, nbytes) == 0
                if shares.value == 1:
                    assert (klen.value, tiles.value, nbytes.value) == (0, 0, 0)
                    continue
                seen_split += 1
                assert klen.value % 32 == 0 and klen.value > 0
                assert klen.value * (shares.value - 1) < K <= klen.value * shares.value    # every share holds some of k
                assert tiles.value == ((M + 63) // 64) * ((N + 63) // 64) <= 4096
                assert nbytes.value == shares.value * tiles.value * 64 * 64 * es <= 128 << 20
                assert first.value == 0                                                    # every tile is split
                if forced is None:      # the automatic choice splits only few tiles with a long k
                    assert tiles.value <= 128 and tiles.value * shares.value <= (1024 if es == 4 else 512)
                    assert K >= (4096 if es == 4 else 2048) and klen.value >= 8 * 32
    assert seen_split >= 10
    # left-over tiles as a tail: whole rounds (a round = the tiles resident at once: 256 units x 2 or 3
    # work-groups) stay unsplit, the rest is split; the automatic plan needs a whole round in the body
    for name, (bm, bn, occ) in ((b"mfma_f32_256x128t", (256, 128, 2)), (b"mfma_f32_128x128t", (128, 128, 3))):
        for (M, N, K) in [(4097, 4095, 4093), (8191, 8193, 8190), (5000, 5000, 5000), (4096, 4096, 4096), (300, 200, 100),
                          (7168, 7168, 7168), (3000, 3000, 64), (100000, 128, 4096)]:
            shares, klen, first, tiles, nbytes = u32(), u32(), u64(), u64(), sz()
            assert lib.wk_gemm_split_plan(8, 0, 0, M, N, K, name, shares, klen, first, tiles, nbytes) == 0
            total = ((M + bm - 1) // bm) * ((N + bn - 1) // bn)
            if shares.value == 1:
                continue
            assert first.value % (256 * occ) == 0 and first.value + tiles.value == total and 0 < tiles.value < 256 * occ
            assert klen.value % 16 == 0 and klen.value * (shares.value - 1) < K <= klen.value * shares.value
            assert nbytes.value == shares.value * tiles.value * bm * bn * 4 <= 128 << 20 and tiles.value <= 4096
    shares, klen, first, tiles, nbytes = u32(), u32(), u64(), u64(), sz()
    assert lib.wk_gemm_split_plan(8, 0, 0, 512, 512, 8192, b"mfma_f64_64x64z", shares, klen, first, tiles, nbytes) == 1   # wrong dtype
    assert lib.wk_gemm_split_plan(8, 0, 0, 512, 512, 8192, b"nope", shares, klen, first, tiles, nbytes) == 1
    assert lib.wk_gemm_split_plan(8, 0, 0, 0, 512, 8192, None, shares, klen, first, tiles, nbytes) == 1


def _split_args(arglist):
    """Top-level comma split of a parameter list (brackets of `[3]u64`, `[*:0]const u8` stay whole)."""
    out, depth, cur = [], 0, ""
    for ch in arglist:
        if ch in "([":
            depth += 1
        elif ch in ")]":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip() and cur.strip() != "void":
        out.append(cur)
    return out


def test_thin_products_and_strips_by_name():
    """Host arithmetic of the launch plan, through the name query (256 compute units and 16-byte aligned
    operands assumed): which f32 / f64 products run as thin products, which are launched as a body of whole
    tiles plus strips, and which stay whole."""
    from wekua_amd import _capi
    lib = _capi.load()

    def name(dtype, M, N, K, op_a=0, op_b=0, lda=None, ldb=None):
        lda = lda or (M if op_a else K)
        ldb = ldb or (K if op_b else N)
        return lib.wk_gemm_variant(dtype, op_a, op_b, M, N, K, lda, ldb, N, None, None, None).decode()
    for dt in (8, 9):
        per = 4 if dt == 8 else 2
        for op_a, op_b in ((0, 0), (0, 1), (1, 0), (1, 1)):
            # at most four rows or four columns, the other dimension and k long enough
            assert name(dt, 1, 4096, 4096, op_a, op_b) == "thin" and name(dt, 4096, 4, 512, op_a, op_b) == "thin"
            assert name(dt, 5, 4096, 4096, op_a, op_b) != "thin" and name(dt, 1, 256, 4096, op_a, op_b) != "thin"
            assert name(dt, 4, 4, 4096, op_a, op_b) != "thin" and name(dt, 1, 4096, 64, op_a, op_b) != "thin"
            # two to 32 rows or columns against a large operand whose rows start on 16-byte boundaries: the kernel
            # that streams that operand once
            assert name(dt, 5, 4096, 4096, op_a, op_b) == "skinny" and name(dt, 4, 4096, 4096, op_a, op_b) == "skinny"
            assert name(dt, 4096, 32, 4096, op_a, op_b) == "skinny" and name(dt, 65, 4096, 4096, op_a, op_b) != "skinny"
            assert name(dt, 32, 4096, 512, op_a, op_b) != "skinny" and name(dt, 32, 200, 65536, op_a, op_b) != "skinny"
            assert name(dt, 16, 4095, 4095, op_a, op_b, ldb=4095) != "skinny"
            # 33 to 64: only with a large operand that is contiguous along the long side (f32: and a short one along k)
            assert (name(dt, 64, 4096, 4096, op_a, op_b) == "skinny") == (op_b == 0 and (op_a == 0 or dt == 9))
            assert (name(dt, 4096, 48, 4096, op_a, op_b) == "skinny") == (op_a == 1 and (op_b == 1 or dt == 9))
            lda, ldb = (4100 if op_a else 4096), (4096 if op_b else 4100)
            assert name(dt, 4097, 4097, 4096, op_a, op_b, lda, ldb).endswith("+strips")
            assert name(dt, 4097, 4097, 4095, op_a, op_b, 4097 if op_a else 4095, 4095 if op_b else 4097).endswith("+strips")
            assert not name(dt, 4096, 4096, 4096, op_a, op_b).endswith("+strips")              # nothing beyond
            assert not name(dt, 4097, 4096, 256, op_a, op_b, lda, 4096).endswith("+strips")     # short k
            assert not name(dt, 1025, 1024, 4096, op_a, op_b, 1028 if op_a else 4096, 4096 if op_b else 1024).endswith("+strips")  # small body
    assert lib.wk_test_option(b"skinny", 0) == 0
    try:
        assert name(8, 5, 4096, 4096) != "skinny" and name(8, 4, 4096, 4096) == "thin"
    finally:
        lib.wk_test_option(b"skinny", 1)
    assert name(4, 4097, 4097, 4096) in ("mfma_i32_128x128", "mfma_i32_64x128")            # integers: never in parts
    assert name(8, 4200, 4096, 1024).endswith("+strips") and not name(8, 3000, 3000, 1024, lda=3000, ldb=3000).endswith("+strips")


ZIG_BINDING = os.path.join(ROOT, "zig", "src", "core", "hip.zig")


def test_zig_binding_matches_the_header():
    """zig/src/core/hip.zig, the `extern fn` block a wekua maintainer drops into src/core, declares exactly
    the functions of the product header, each with the header's number of parameters (no Zig toolchain
    exists here to compile it, so this is the check it gets), and none of the test knobs."""
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    header = {m.group(1): len(_split_args(m.group(2)))
              for m in re.finditer(r"\b(wk_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S)}
    src = re.sub(r"//[^\n]*", "", open(ZIG_BINDING).read())
    zig = {m.group(1): len(_split_args(m.group(2)))
           for m in re.finditer(r"pub extern fn (wk_[a-z0-9_]+)\(([^;]*?)\)\s*[^;()]*;", src, flags=re.S)}
    assert set(header) == set(declared_functions((HEADER,)))
    assert set(zig) == set(header), f"not in hip.zig: {set(header) - set(zig)}; not in the header: {set(zig) - set(header)}"
    wrong = {n: (header[n], zig[n]) for n in header if header[n] != zig[n]}
    assert not wrong, f"parameter counts differ (header, hip.zig): {wrong}"
    # the rewritten call sites only use what the binding declares
    zig_dir = os.path.join(ROOT, "zig", "src")
    for dirpath, _dirs, files in os.walk(zig_dir):
        for f in files:
            used = set(re.findall(r"hip\.(wk_[a-z0-9_]+)", open(os.path.join(dirpath, f)).read()))
            assert used <= set(zig), f"{f} calls undeclared {used - set(zig)}"


def test_header_compiles_as_plain_c():
    """The boundary is a C ABI: the header must be valid C, not only C++."""
    src = '#include "wekua_hip.h"\nint main(void){ int (*f)(wk_stream*, int, int, int, uint64_t, uint64_t, uint64_t, const void*, const void*, uint64_t, const void*, uint64_t, const void*, void*, uint64_t, void*, size_t) = wk_gemm; return f != wk_gemm; }\n'
    res = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                          "-x", "c", "-"], input=src, text=True, capture_output=True)
    assert res.returncode == 0, res.stderr


def test_host_only_entry_points():
    from wekua_amd import _capi
    lib = _capi.load()
    assert lib.wk_abi_version() == 1
    sizes = [lib.wk_dtype_size(i) for i in range(20)]
    assert sizes == [1, 1, 2, 2, 4, 4, 8, 8, 4, 8, 2, 2, 4, 4, 8, 8, 16, 16, 8, 16]
    assert lib.wk_dtype_size(20) == 0 and lib.wk_dtype_size(-1) == 0
    # error names are the reference's Zig error names (src/tensor/main.zig:25-33)
    names = {1: "InvalidValue", 2: "InvalidCoordinates", 3: "InvalidBuffer", 4: "UnqualTensorsAttribute",
             5: "UnqualTensorsShape", 6: "UnqualTensorsDimension", 7: "UnqualTensorsContext", 8: "OutOfMemory",
             9: "TypeNotSupported", 10: "DevicesArrayEmpty"}
    for code, name in names.items():
        assert lib.wk_strerror(code).decode() == name
    assert lib.wk_strerror(11).decode().startswith("ScratchTooSmall")
    assert lib.wk_gemm_workspace_bytes(8, 0, 0, 8192, 8192, 8192) == 0
    assert lib.wk_gemm_force_variant(b"no-such-kernel") == 1
    assert lib.wk_gemm_force_variant(b"auto") == 0
    # kernel selection is host logic: f32/f64 and the 32-bit integers go to the matrix cores (the
    # integers through their int8 decomposition), everything else to the tile kernel
    v = lambda dt, n: lib.wk_gemm_variant(dt, 0, 0, n, n, n, n, n, n, None, None, None).decode()
    assert v(8, 8192).startswith("mfma_f32")
    assert v(9, 4096).startswith("mfma_f64")
    assert v(4, 2048) == "mfma_i32_128x128" and v(5, 2048) == "mfma_u32_128x128" and v(4, 1024) == "mfma_i32_64x128"
    assert v(2, 2048) == "tile64" and v(6, 2048) == "tile64" and v(14, 512) == "tile64"
    assert v(18, 512) == "tile64"
    assert lib.wk_gemm_variant(8, 0, 0, 0, 4, 4, 4, 4, 4, None, None, None).decode() == "invalid"


def _gpu_present():
    from wekua_amd import _capi
    n = ctypes.c_int(-1)
    assert _capi.load().wk_device_count(ctypes.byref(n)) == 0
    return n.value > 0


def test_no_gpu_means_loud_failure_not_fallback():
    """Without a device the product path raises DevicesArrayEmpty (src/core/context.zig:18); it
    never computes on the host."""
    if _gpu_present():
        pytest.skip("a GPU is present")
    import wekua_amd
    with pytest.raises(wekua_amd.WekuaError) as e:
        wekua_amd.Context.initFromDeviceType(wekua_amd.DeviceType.all)
    assert e.value.name == "DevicesArrayEmpty"
    from wekua_amd import raw
    with pytest.raises(wekua_amd.WekuaError):
        raw.Device(0)


def test_product_package_never_touches_the_oracle():
    """The GPU package must not import, load or link anything under oracle/."""
    pkg = os.path.join(ROOT, "wekua_amd")
    for dirpath, _dirs, files in os.walk(pkg):
        if os.path.basename(dirpath) in ("build", "__pycache__"):
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "wk_oracle" not in text and "import oracle" not in text and "from oracle" not in text, f
    for so in ("libwekua_hip.so", "libwekua_host.so"):
        out = subprocess.run(["ldd", os.path.join(pkg, so)], capture_output=True, text=True).stdout
        assert "oracle" not in out
