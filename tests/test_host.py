"""Host-side logic without a GPU: the C-ABI library loads and exports what include/descent_hip.h declares, the
code generator produces gfx950-compilable HIP for every kernel kind (hipRTC needs no device), the graph passes
reproduce the reference's cluster structure, and error paths answer with errors instead of crashes."""
import ctypes as C
import json
import os
import re

import numpy as np
import pytest

from descent_amd import Environment, Initializer, _abi, hip_backend, kernel as K, workloads
from descent_amd.shape import BATCHES, Shape, View
from oracle.cpu_backend import CpuBackend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _env():
    return Environment(CpuBackend())


def test_library_exports_every_declared_entry_point():
    header = open(os.path.join(ROOT, "include", "descent_hip.h")).read()
    declared = set(re.findall(r"^(?:int|int64_t|void|const char\*)\s+(dsc_[a-z_0-9]+)\s*\(", header, re.M))
    assert len(declared) >= 30
    lib = C.CDLL(hip_backend.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert declared == set(hip_backend.EXPORTED_SYMBOLS)


def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 with no C++ in it, and a C program that includes it links
    against the library and gets DSC_ERR_NO_DEVICE (here) or a context (on a GPU box) from dsc_ctx_create."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if not gcc:
        pytest.skip("no gcc")
    header_dir = os.path.join(ROOT, "include")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c",
                    os.path.join(header_dir, "descent_hip.h")], check=True)
    src = tmp_path / "probe.c"
    src.write_text(
        '#include "descent_hip.h"\n#include <stdio.h>\n'
        "int main(void) {\n"
        "    dsc_ctx* ctx = 0;\n"
        "    int rc = dsc_ctx_create(0, &ctx);\n"
        '    printf("%d %s\\n", rc, rc ? dsc_last_error() : "ok");\n'
        "    if (rc == 0) dsc_ctx_destroy(ctx);\n"
        "    return 0;\n}\n")
    exe = tmp_path / "probe"
    lib_dir = os.path.dirname(hip_backend.LIB_PATH)
    subprocess.run([gcc, "-std=c99", "-I", header_dir, str(src), "-o", str(exe), "-L", lib_dir, "-ldescent_hip",
                    "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split(None, 1)
    assert int(out[0]) in (0, _abi.ERR_NO_DEVICE), out


def test_no_device_is_an_error_not_a_fallback():
    """This container has no GPU: creating a context must fail with DSC_ERR_NO_DEVICE."""
    lib = hip_backend.lib()
    ctx = C.c_void_p()
    rc = lib.dsc_ctx_create(0, C.byref(ctx))
    if rc == 0:  # running on a GPU box
        lib.dsc_ctx_destroy(ctx)
        pytest.skip("a GPU is present")
    assert rc == _abi.ERR_NO_DEVICE and not ctx.value
    with pytest.raises(hip_backend.DescentHipError):
        hip_backend.HipBackend()


def _kernels_of_each_kind():
    sh = Shape((4, 6, 8))
    ident = sh.identity_view()
    pe = K.PerElementKernel(
        192,
        (ident, View.broadcast(Shape((8,)), sh)),
        (6,),
        (K.PeLoad(0), K.PeLoad(1), K.PeBinary("Add", (0, 1)), K.PeLiteral(K.Literal.f32(0.0)),
         K.PeLiteral(K.Literal.f32(0.01)), K.PeBinary("Mul", (2, 4)), K.PeSelect("Gt", (2, 3, 2, 5))),
    )
    pe_rand = K.PerElementKernel(
        192, (ident,), (4,),
        (K.PeLoad(0), K.PeRand(3, ident), K.PeCoord(View.broadcast(Shape((1, 1, 8)), sh)), K.PeBinary("Mul", (0, 1)),
         K.PeBinary("Add", (3, 2))),
    )
    gather_shape = Shape((4, 10, 8))
    pe_gather = K.PerElementKernel(
        320, (ident, View.broadcast(Shape((1, 10, 1)), gather_shape)), (1,),
        (K.PeLoad(1), K.PeGather(gather_shape, 1, 0, 0)),
    )
    win = Shape((2, 3, 3, 1, 2, 2, 4))
    return [
        K.FillKernel(K.Literal.f32(1.5), 1000),
        K.FillKernel(K.Literal.u32(7), 1001),
        pe, pe_rand, pe_gather,
        K.ReduceKernel(sh.reduce(2), ident, "Sum", 2),
        K.ReduceKernel(sh.reduce(0), ident, "Max", 0),
        K.MatMulKernel(Shape((1, 4, 6, 5)), BATCHES, ident, Shape((4, 8, 5)).identity_view()),
        K.MatMulKernel(Shape((2, 1, 300, 200)), BATCHES, Shape((1, 300, 1100)).identity_view(),
                       Shape((1, 200, 1100)).identity_view().transposed()),
        K.UnpadKernel(Shape((4, 2, 8)), ident, 1, 2),
        K.WindowsToImageKernel(Shape((2, 6, 6, 4)), win.identity_view(), (2, 2)),
        K.ScatterAddKernel(Shape((4, 9, 8)), ident, 1, Shape((6,)).identity_view()),
    ]


@pytest.mark.parametrize("kernel", _kernels_of_each_kind(), ids=lambda k: type(k).__name__)
def test_generated_source_compiles_for_gfx950(kernel):
    src = hip_backend.codegen_source(kernel)
    assert 'extern "C" __global__' in src and re.search(r"void (dsc_[a-z_0-9]+|MM_ENTRY)\(", src)
    assert hip_backend.codegen_compile(kernel, "gfx950") > 0
    if isinstance(kernel, K.MatMulKernel):
        assert "__builtin_amdgcn_mfma_f32_32x32x2f32" in src
    if isinstance(kernel, K.ScatterAddKernel):
        assert "unsafeAtomicAdd" in src


def test_malformed_descriptors_are_rejected_with_a_message():
    sh = Shape((4, 6))
    bad = [
        K.PerElementKernel(24, (sh.identity_view(),), (1,), (K.PeLoad(0), K.PeUnary("Exp", 1))),  # arg not earlier
        K.PerElementKernel(24, (sh.identity_view(),), (5,), (K.PeLoad(0),)),                      # missing output op
        K.PerElementKernel(25, (sh.identity_view(),), (0,), (K.PeLoad(0),)),                      # element count
        K.ReduceKernel(Shape((4, 6)), sh.identity_view(), "Sum", 1),                              # axis not collapsed
        K.MatMulKernel(Shape((1, 1, 4, 5)), BATCHES, Shape((1, 4, 6)).identity_view(), Shape((1, 7, 5)).identity_view()),
        K.UnpadKernel(Shape((4, 6)), sh.identity_view(), 1, 1),
    ]
    for kernel in bad:
        with pytest.raises(hip_backend.DescentHipError) as e:
            hip_backend.codegen_source(kernel)
        assert e.value.status == _abi.ERR_INVALID and len(str(e.value)) > 20


def test_tensors_beyond_32_bit_indexing_are_refused_not_wrapped():
    """Kernels index with 32-bit integers: a descriptor whose output or any input reaches 2^31 elements is refused
    with DSC_ERR_UNSUPPORTED; the largest size below the limit still generates."""
    big = Shape((32768, 65536))
    edge = Shape((32768, 65535))
    over = [
        K.PerElementKernel(big.element_count(), (big.identity_view(),), (1,), (K.PeLoad(0), K.PeUnary("Exp", 0))),
        K.ReduceKernel(Shape((1, 65536)), big.identity_view(), "Sum", 0),
        K.MatMulKernel(Shape((1, 1, 8, 8)), BATCHES, Shape((1, 8, 1 << 28)).identity_view(), Shape((1, 1 << 28, 8)).identity_view()),
        K.FillKernel(K.Literal.f32(0.0), 1 << 31),
    ]
    for kernel in over:
        with pytest.raises(hip_backend.DescentHipError) as e:
            hip_backend.codegen_source(kernel)
        assert e.value.status == _abi.ERR_UNSUPPORTED and "32-bit" in str(e.value), str(e.value)
    ok = K.PerElementKernel(edge.element_count(), (edge.identity_view(),), (1,), (K.PeLoad(0), K.PeUnary("Exp", 0)))
    assert "dsc_per_element_n2147450880" in hip_backend.codegen_source(ok)


def test_array_api_cluster_structure_matches_the_reference_dumps():
    """docs/array_api_values.svg / array_api_grad.svg of the reference, reduced to JSON by
    tests/golden/make_array_api_fixture.py."""
    want = json.load(open(os.path.join(ROOT, "tests", "golden", "array_api_clusters.json")))
    env = _env()
    m = env.static_parameter([3, 3], "m")
    x = env.static_parameter([3, 1], "x")
    y = env.static_parameter([3, 1], "y")
    z = env.static_parameter([3, 1], "z")

    def values(s):
        mv, xv, yv = s.parameter_value(m), s.parameter_value(x), s.parameter_value(y)
        s.write_parameter_value(z, 2.0 * mv.matmul(xv) + yv * yv + 1.0)

    xp = env.trainable_parameter([1], "x", Initializer.zero())

    def grad(s):
        xd = s.parameter(xp)
        yd = xd.sin()
        (yd.square() + yd * 3.0).set_loss()
        s.write_parameter_value(xp, xd.value() - 0.1 * xd.loss_grad())

    for key, build in (("values", values), ("grad", grad)):
        g = env.build_graph(build)
        got = []
        for cid in g.clusters_sorted:
            k = g.clusters[cid].kernel
            if isinstance(k, K.MatMulKernel):
                got.append(["MatMul"])
            else:
                labels = []
                for op in k.ops:
                    if isinstance(op, (K.PeUnary, K.PeBinary)):
                        labels.append(op.op)
                got.append(sorted(labels))
        assert sorted(got) == want[key]["clusters"], key
        # literals are inlined into the cluster as the dumps show them outside any kernel node
        n_literals = sum(1 for lab in want[key]["outside"] if re.fullmatch(r"-?\d+E-?\d+", lab))
        pe = [g.clusters[c].kernel for c in g.clusters_sorted if isinstance(g.clusters[c].kernel, K.PerElementKernel)][0]
        assert sum(isinstance(op, K.PeLiteral) for op in pe.ops) == n_literals


def test_convnet_graph_shape():
    env = _env()
    w = workloads.convnet(env, batch=1000)
    labels = w.graph.kernel_labels()
    assert len(labels) == 66
    # the GEMMs the train step contains, with the reference's split-K factors r = ceil(K/1024)
    for want in ["MatMul (k=9) [1, 784000, 1, 16]", "MatMul (k=784000) [766, 1, 9, 16]", "MatMul (k=72) [1, 196000, 2, 16]",
                 "MatMul (k=196000) [192, 2, 72, 16]", "MatMul (k=16) [1, 2, 196000, 72]", "MatMul (k=1568) [2, 1, 1000, 128]",
                 "MatMul (k=1000) [1, 1, 1568, 128]", "MatMul (k=128) [1, 1, 1000, 1568]", "MatMul (k=128) [1, 1, 1000, 10]",
                 "MatMul (k=1000) [1, 1, 128, 10]", "MatMul (k=10) [1, 1, 1000, 128]"]:
        assert want in labels, want
    assert sum(p.shape.element_count() for p in w.trainable) == 204618
    listing = hip_backend.check_schedule(w.graph, fused=True)
    launches = int(listing.split()[0])
    assert launches < 30, listing
    # the classifier head (1000 x 128 -> 10), softmax cross-entropy and the accuracy count: one row-fused launch over the
    # [1000, 10] logits, whose first stage is the MatMul (the lanes of a row share its k range)
    assert "RowFused [1000, 10] (10 clusters)" in listing
    assert "10 stages, the first a MatMul over k=128 shared by the row's lanes" in listing
    # small independent launches (optimiser updates of small tensors, short reductions) share launches
    assert listing.count("Multi (") >= 3
    # every reference cluster is covered exactly once, except producers inlined into several consumers
    covered = [int(c) for line in listing.splitlines() if " clusters " in line for c in line.split(" clusters ")[1].split()]
    assert set(covered) == set(range(66))
    # the data gradient of the second convolution: MatMul + reshape copy + WindowsToImage as one product over
    # the padded image, both operands fused producers
    assert "ConvBackward" in listing and "data gradient 3x3 taps x 16 channels with border folds, filter gradient mfma 16x16x4 5x1 tiles +column sums of dC" in listing
    split = hip_backend.check_schedule(w.graph, fused="split-conv-grads")
    assert "ConvDataGrad" in split and "conv data gradient: workgroup per image and group, tile in LDS, 3x3 taps x 16 channels, border folds fused" in split
    assert "tall-k mfma 16x16x4, 5x1 tiles" in split and "ConvBackward" not in split
    # on its own the same product is the dot-product kernel: lanes share a row's k range, no MFMA tile grid of 32
    # single-wave workgroups
    head = workloads.matmul_epilogue(_env(), 1000, 10, 128, upload=False)
    assert "[dot products: 16 lanes per row, B in LDS +epilogue]" in hip_backend.check_schedule(head.graph, fused=True)
    # both forward convolutions: the image tile goes to LDS, the im2col copy stays only for the filter gradient
    assert listing.count("ConvForward") == 2
    assert "conv forward: workgroup per image and group, padded image tile in LDS, mfma 16x16x4, 3x3 taps x 8 channels +epilogue" in listing
    generic = hip_backend.check_schedule(w.graph, fused="generic-conv")
    assert "MatMul (k=144) [1, 256000, 2, 8]" in generic and "ConvForward" not in generic and "ConvDataGrad" not in generic
    # the work figures of the listing: the eleven GEMMs of the step as the reference runs them
    assert "4.373 GFLOP in MatMuls" in hip_backend.check_schedule(w.graph, fused=False)


def test_work_figures_of_the_headline_matmul():
    env = _env()
    w = workloads.matmul_epilogue(env, 8192, 8192, 8192, upload=False)
    listing = hip_backend.check_schedule(w.graph, fused=True)
    assert int(listing.split()[0]) == 1
    # 4 * (M*K + K*N + N + M*N) bytes and 2*M*N*K flops
    assert "805.339 MB moved, 1099.512 GFLOP" in listing, listing


def test_fused_and_unfused_schedules_compile_for_every_config():
    env = _env()
    graphs = [workloads.convnet(env, batch=8).graph, workloads.linear_classifier(env, batch=16).graph,
              workloads.matmul_epilogue(env, 300, 200, 1100, upload=False).graph]
    for g in graphs:
        fused = hip_backend.check_schedule(g, fused=True)
        unfused = hip_backend.check_schedule(g, fused=False)
        assert int(unfused.split()[0]) == len(g.clusters_sorted)
        assert int(fused.split()[0]) <= int(unfused.split()[0])


def test_reference_error_behaviour_on_the_host():
    env, other = _env(), _env()
    p = other.static_parameter([4], "p")
    with pytest.raises(ValueError, match="same environment"):  # src/parameter.rs:51-56
        env.build_graph(lambda s: s.parameter_value(p))
    q = env.static_parameter([4], "q")
    r = env.static_parameter([5], "r")
    env.write_parameter(r, np.zeros(5, np.float32))
    with pytest.raises(ValueError, match="shape mismatch"):  # src/array.rs:1367-1370
        env.build_graph(lambda s: s.write_parameter_value(q, s.parameter_value(r)))
    with pytest.raises(ValueError):  # src/shape.rs:97-98
        Shape((1, 4, 5)).batched_matmul(Shape((1, 6, 3)), BATCHES)
    with pytest.raises(ValueError, match="no value"):  # src/environment.rs:375 (assert on missing buffer)
        env.run(env.build_graph(lambda s: s.write_parameter_value(q, s.parameter_value(q) + 1.0)), 0)


def test_writer_zero_fills_the_unwritten_tail():
    env = _env()
    p = env.static_parameter([8], "p")
    with env.writer(p) as w:
        w.write(np.arange(3, dtype=np.float32))
    assert np.array_equal(env.read_parameter_to_vec(p), np.array([0, 1, 2, 0, 0, 0, 0, 0], np.float32))


def test_parameters_round_trip_through_a_raw_f32_file(tmp_path):
    env = _env()
    rng = np.random.default_rng(1)
    shapes = ([3, 5], [7], [2, 2, 2])
    params = [env.static_parameter_with_data(sh, f"p{i}", rng.standard_normal(sh, dtype=np.float32)) for i, sh in enumerate(shapes)]
    before = [env.read_parameter(p) for p in params]
    path = tmp_path / "params.f32"
    assert env.save_parameters(path, params) == 4 * (15 + 7 + 8)
    assert np.array_equal(np.fromfile(path, dtype="<f4"), np.concatenate([b.ravel() for b in before]))
    for p in params:
        env.writer(p).zero_fill()
    env.load_parameters(path, params)
    for p, b in zip(params, before):
        assert np.array_equal(env.read_parameter(p), b)
    with pytest.raises(ValueError, match="bytes"):
        env.load_parameters(path, params[:2])


def test_image_fit_parameter_counts_match_the_reference_readme():
    """examples/image_fit/README.md:31-34: ReLU 44099, ReLU-PE 51779, SIREN 44099, MULTI-HASH 43977 trainable
    parameters for hidden units [256,128,64,32], 8 frequencies, and 10 levels from 2 to 512 with 4096 entries."""
    env = _env()
    hidden = (256, 128, 64, 32)
    count = lambda m: sum(p.shape.element_count() for p in [q for layer in m.hidden + [m.final] for q in (layer.w, layer.b)])
    assert count(workloads.ReluMlp(env, 0, hidden)) == 44099
    assert count(workloads.ReluMlp(env, 8, hidden)) == 51779
    assert count(workloads.Siren(env, hidden)) == 44099
    b = np.exp((np.log(np.float32(512)) - np.log(np.float32(2))) / np.float32(9)).astype(np.float32)
    sizes = [int(np.float32(2) * b ** np.float32(i)) for i in range(10)]
    mh = workloads.MultiHashGrid(env, sizes, 4096, (64, 64))
    total = count(mh) + sum(g.t.shape.element_count() for g in mh.grids)
    assert total == 43977, (total, sizes)


def test_code_object_cache_hit_miss_and_damaged_files(tmp_path, monkeypatch):
    """The on-disk code-object cache through the device-free compile path: a miss compiles and writes a file, a hit
    uses it without calling hipRTC, and a truncated, a bit-flipped and a foreign file are each deleted and the kernel
    compiled again (the counterpart of the reference's per-process KernelCache, src/kernel.rs:1037-1056)."""
    cache = tmp_path / "cache"
    cache.mkdir()
    monkeypatch.setenv("DSC_CACHE_DIR", str(cache))
    kernel = K.FillKernel(K.Literal.f32(2.25), 4321)

    def compile_once():
        before = hip_backend.cache_stats()
        size = hip_backend.codegen_compile(kernel)
        after = hip_backend.cache_stats()
        return size, tuple(a - b for a, b in zip(after, before))

    size, delta = compile_once()
    assert delta == (0, 1, 0)  # miss: one hipRTC compilation
    files = list(cache.iterdir())
    assert len(files) == 1 and files[0].suffix == ".co"
    blob = files[0].read_bytes()
    assert blob[:8] == b"DSCCOBJ2" and blob[24:28] == b"\x7fELF" and len(blob) == 24 + size

    size2, delta = compile_once()
    assert (size2, delta) == (size, (1, 0, 0))  # hit: the file, no compilation

    damaged = {
        "truncated": blob[: len(blob) // 2],
        "one bit flipped in the payload": blob[:1000] + bytes([blob[1000] ^ 0x10]) + blob[1001:],
        "not a cache file": b"\x7fELF" + b"\0" * 4096,
        "header only": blob[:24],
        "right header, payload is not a code object": None,
    }
    junk = b"#!/bin/sh\n" * 100
    import struct

    def fnv(data):
        h = 1469598103934665603
        for byte in data:
            h = ((h ^ byte) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
        return h

    damaged["right header, payload is not a code object"] = b"DSCCOBJ2" + struct.pack("<QQ", len(junk), fnv(junk)) + junk
    for what, data in damaged.items():
        files[0].write_bytes(data)
        size3, delta = compile_once()
        assert (size3, delta) == (size, (0, 1, 1)), what  # refused, deleted, compiled again
        assert files[0].read_bytes() == blob, what         # and the cache holds a good file again

    # the key covers the compile options and tool versions: another kernel is another file
    hip_backend.codegen_compile(K.FillKernel(K.Literal.f32(2.25), 4322))
    assert len(list(cache.iterdir())) == 2

    monkeypatch.setenv("DSC_CACHE_DIR", "off")
    _, delta = compile_once()
    assert delta == (0, 1, 0) and len(list(cache.iterdir())) == 2


def test_every_environment_variable_the_library_reads_is_documented():
    read = set()
    csrc = os.path.join(ROOT, "descent_amd", "csrc")
    for name in os.listdir(csrc):
        if name.endswith((".cpp", ".hpp")):
            read |= set(re.findall(r'getenv\("(DSC_[A-Z_0-9]+)"\)', open(os.path.join(csrc, name)).read()))
            # names reached through a loop over a list of strings
            read |= set(re.findall(r'"(DSC_(?:MM|ROWS|FUSE)_[A-Z_0-9]+)"', open(os.path.join(csrc, name)).read()))
    assert len(read) >= 15
    documented = set(re.findall(r"`(DSC_[A-Z_0-9]+)", open(os.path.join(ROOT, "INTEGRATION.md")).read()))
    assert read <= documented, sorted(read - documented)
