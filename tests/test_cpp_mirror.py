"""The C header is plain C99 and the C++ host mirror compiles against it (syntax and linkage only)."""
import os
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no gcc")
def test_header_is_c99():
    src = '#include "ctinytitan_hip.h"\nint main(void) { return (int)sizeof(tt_half) - 2; }\n'
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "t.c")
        open(path, "w").write(src)
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic-errors", "-I", INC, "-c", path,
                        "-o", os.path.join(d, "t.o")], check=True)


@pytest.mark.skipif(shutil.which("g++") is None, reason="no g++")
def test_cpp_mirror_compiles_and_links():
    from tinytitan_amd import capi
    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("library not built")
    src = r'''
#include "TinyTitanHIP.hpp"
#include <cstdio>
int main() {
    // host arithmetic first: the reference's row-layout known answers (KVCacheQuantizedAttentionTests.swift:96-98)
    if (tinytitan::KVCacheManager::rowLayout(512, tinytitan::KVCachePrecision::int8).first != 544) return 2;
    if (tinytitan::KVCacheManager::rowLayout(512, tinytitan::KVCachePrecision::int4).first != 288) return 2;
    if (tinytitan::KVCacheManager::rowLayout(512, tinytitan::KVCachePrecision::fp16).second != 1024) return 2;
    // the dense-exact window of the sparse attention (QSAExactnessTests.swift:14-36, :82-91)
    const tinytitan::QSAExactness production(2048, 4);
    if (production.keptBlocks() != 512 || production.maximumExactVisibleKeys() != 2051) return 4;
    if (!production.isDenseExact(2051) || production.isDenseExact(2052) || production.indexerRequiredFromContext() != 2052) return 4;
    if (tinytitan::QSAExactness(64, 1).maximumExactVisibleKeys() != 64 || tinytitan::QSAExactness(512, 8).maximumExactVisibleKeys() != 64 * 8 + 7) return 4;
    try {
        tinytitan::Context ctx(0);
        tinytitan::KVCacheManager kv(ctx, 1, 2, 256, 1, 4096);
        std::printf("capacity %d stride %zu\n", kv.capacityTokens(), kv.strideBytes());
        tinytitan::KVCacheManager kv8(ctx, 1, 2, 256, 1, 4096, 0, tinytitan::KVCachePrecision::int8);
        if (kv8.strideBytes() != 544 || kv8.precision() != tinytitan::KVCachePrecision::int8) return 3;
        tinytitan::QSAIndexer indexer(ctx, 4, 128, 4, 64, 1e7f);
        if (indexer.selectionWidth() != 67) return 5;  // QSAIndexerTests.swift:47
        if (indexer.encodeSelectKeys(nullptr, 0, 1, 67, nullptr, 0)) return 5;  // inside the window: no selection, nothing touched
    } catch (const tinytitan::Error &e) {
        std::printf("status %d\n", e.status());
        return e.status() == TT_HIP_ERR_NO_DEVICE ? 0 : 1;
    }
    return 0;
}
'''
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "t.cpp")
        open(path, "w").write(src)
        exe = os.path.join(d, "t")
        libdir = os.path.dirname(capi.LIB_PATH)
        subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I", INC, path, "-o", exe, "-L", libdir,
                        "-lctinytitan_hip", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"], check=True)
        out = subprocess.run([exe], capture_output=True, text=True)
        assert out.returncode == 0, out.stdout + out.stderr
