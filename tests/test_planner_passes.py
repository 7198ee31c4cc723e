"""One small graph per pass of the fusion planner (descent_amd/csrc/schedule.cpp, struct Planner), planned and compiled
for gfx950 without a GPU; each test reads the listing for the launches the pass must have produced, next to the
cluster-by-cluster listing of the same graph.  The convolution passes, the row-fused launch and the max-pool fusion
are read off the ConvNet's listing in test_host.py."""
import os
import re
import subprocess
import sys

from descent_amd import Environment, hip_backend, workloads
from oracle.cpu_backend import CpuBackend


def _env():
    return Environment(CpuBackend())  # graphs are only built and planned here, never run


def _listings(shapes, build):
    env = _env()
    params = [env.static_parameter(s, f"p{i}") for i, s in enumerate(shapes)]
    graph = env.build_graph(lambda scope: build(scope, *params))
    unfused = hip_backend.check_schedule(graph, fused=False)
    assert int(unfused.split()[0]) == len(graph.clusters_sorted)
    return unfused, hip_backend.check_schedule(graph, fused=True)


def _value(scope, p):
    return scope.parameter_value(p)


def _chunks(listing):
    return [int(c) for c in re.findall(r"chunks (\d+)", listing)]


def test_a_long_k_over_a_small_product_is_split_over_more_workgroups():
    unfused, fused = _listings([[8, 200000], [200000, 16], [8, 16]],
                               lambda s, a, b, c: s.write_parameter_value(c, _value(s, a).matmul(_value(s, b))))
    # the reference's ceil(k / 1024) chunks against a split that fills 256 compute units
    assert _chunks(unfused) == [196]
    assert _chunks(fused)[0] >= 512
    # the partial products are summed by the Reduce the graph already had, which also takes the final copy
    assert int(fused.split()[0]) == 2
    assert re.search(r"Reduce \(k=\d+\) \[1, 1, 8, 16\] \+ PerElement", fused)


def test_a_chain_of_reduces_over_neighbouring_axes_becomes_one_reduce():
    unfused, fused = _listings([[64, 6, 6, 8], [8]], lambda s, x, o: s.write_parameter_value(
        o, _value(s, x).reduce_sum(0, False).reduce_sum(0, False).reduce_sum(0, False)))
    assert unfused.count("Reduce (k=") == 3
    assert int(fused.split()[0]) == 1
    assert "Reduce (k=2304) [1, 1, 1, 8] + PerElement (2 ops) [8]" in fused


def test_a_long_reduce_with_few_outputs_is_split_in_two():
    unfused, fused = _listings([[4, 1 << 20], [4]], lambda s, x, o: s.write_parameter_value(o, _value(s, x).reduce_sum(1, False)))
    assert "Reduce (k=1048576) [4, 1]" in unfused and "grid 1x256" in unfused.splitlines()[1]
    first, second = fused.splitlines()[1:3]
    assert "Reduce (k=512) [4, 2048, 1]" in first and "grid 2048x256" in first
    assert "Reduce (k=2048) [4, 1] + PerElement (2 ops) [4]" in second


def test_light_producers_are_evaluated_inside_the_matmul_that_reads_them():
    unfused, fused = _listings([[512, 512], [512, 512], [512, 512]], lambda s, a, b, c: s.write_parameter_value(
        c, (_value(s, a) * 2.0).matmul(_value(s, b).transpose())))
    assert unfused.splitlines()[1].startswith("0: PerElement (3 ops) [262144]")
    first = fused.splitlines()[1]
    assert first.startswith("0: MatMul (k=512)") and "<1 fused producers>" in first and first.rstrip().endswith("clusters 1 0")


def test_a_reduce_applies_its_only_consumer_before_the_store():
    unfused, fused = _listings([[4096, 256], [256], [256]], lambda s, x, m, o: s.write_parameter_value(
        o, _value(s, m) * 0.9 + _value(s, x).reduce_sum(0, False)))
    assert int(unfused.split()[0]) == 2
    assert "[1, 256] + PerElement (5 ops) [256]" in fused
    assert not any(line.split(": ")[1].startswith("PerElement") for line in fused.splitlines()[1:] if re.match(r"\d+: ", line))


def test_matmul_takes_its_per_element_consumer_as_epilogue():
    w = workloads.matmul_epilogue(_env(), 512, 256, 384, upload=False)
    unfused = hip_backend.check_schedule(w.graph, fused=False)
    fused = hip_backend.check_schedule(w.graph, fused=True)
    assert int(unfused.split()[0]) == len(w.graph.clusters_sorted) >= 2
    assert int(fused.split()[0]) == 1 and "+epilogue" in fused


def test_bias_gradient_rides_on_the_weight_gradient_that_reads_the_same_array():
    graph = workloads.convnet(_env(), batch=1000).graph
    listing = hip_backend.check_schedule(graph, fused="split-conv-grads")
    # conv1: filter gradient im2col^T x dC with the column sums of dC (the bias gradient) from the same pass
    assert re.search(r"MatMul \(k=784000\) \[\d+, 1, 9, 16\] <1 fused producers>  \[tall-k mfma 16x16x4.*\+column sums of B\]", listing)
    assert re.search(r"Reduce \(k=\d+\) \[1, 1, 1, 16\]; Reduce \(k=\d+\) \[1, 1, 9, 16\]", listing)


def _convnet_plan(fused="True", **env):
    """The ConvNet's schedule listing from a process of its own (the planner reads its switches once per process)."""
    code = "import sys; sys.path.insert(0, %r); from descent_amd import Environment, hip_backend, workloads; from oracle.cpu_backend import CpuBackend; " \
           "print(hip_backend.check_schedule(workloads.convnet(Environment(CpuBackend()), batch=1000).graph, fused=%s))"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    return subprocess.run([sys.executable, "-c", code % (root, fused)], env=dict(os.environ, **env), check=True, capture_output=True, text=True).stdout


def test_first_layer_filter_gradient_takes_the_pooling_gradient_as_a_producer():
    listing = _convnet_plan(DSC_POOL_WORDS="0")
    assert int(listing.split()[0]) == 8
    # conv2's backward kernel runs with loader waves and takes its dC the same way: the pooling gradient behind it is
    # a producer of that kernel's fills and no launch of its own
    line = next(l for l in listing.splitlines() if ": ConvBackward" in l)
    assert "fused producers>" in line and "loader waves fill the next image's tiles" in line and "grid 512x512" in line, line
    # conv1 needs no data gradient: its filter gradient (and the bias gradient's column sums) run on the convolution
    # backward kernel, bands of 7 output rows; dC is never written -- the max-pool gradient (a WindowsToImage over
    # 2x2 windows that do not overlap, turned into a copy), the selects around it and the activation derivative are
    # evaluated where the kernel fills its dC tile
    line = next(l for l in listing.splitlines() if "ConvFilterGrad" in l)
    assert "no data gradient, 4 bands of 7 output rows, filter gradient mfma 16x16x4 1x1 tiles +column sums of dC" in line, line
    for cluster in (44, 45, 46, 50):  # select_eq, WindowsToImage, leaky', the filter gradient's MatMul
        assert str(cluster) in line.split(" clusters ")[1].split(), (cluster, line)
    assert "WindowsToImage" not in listing
    assert re.search(r"Reduce \(k=1024\) \[1, 1, 1, 16\]; Reduce \(k=1024\) \[1, 1, 9, 16\]", listing)
    assert "338.4" in listing.strip().splitlines()[-1], listing.strip().splitlines()[-1]
    # with the switch the second convolution keeps its own two kernels and the first its tall-k product
    split = _convnet_plan(fused="'split-conv-grads'")
    assert "ConvFilterGrad" not in split and "ConvBackward" not in split


def test_pooling_gradients_are_read_off_the_window_words_the_forward_kernels_write():
    """Both convolutions' activations are read by nothing but their pooling's and their activation's backward: the
    forward kernels write two bits per element (equals the window's maximum, is positive) in place of the activation,
    the backward kernels read those words and the pooled gradient instead of evaluating four producers."""
    listing = _convnet_plan()
    assert int(listing.split()[0]) == 8
    forward = [l for l in listing.splitlines() if "conv forward:" in l]
    assert len(forward) == 2 and all("window words in place of its source" in l for l in forward), forward
    line = next(l for l in listing.splitlines() if ": ConvBackward" in l)
    assert "dC read off the pooling windows' words" in line and "fused producers" not in line and "loader waves" in line, line
    line = next(l for l in listing.splitlines() if "ConvFilterGrad" in l)
    assert "dC read off the pooling windows' words, no data gradient, 4 bands of 7 output rows" in line, line
    # 75 MB of activations are neither written nor read back; 4.7 MB of words are.  The second convolution's pooled
    # array, which only the pooling's backward read beside the dropout's output, is not written either (6.3 MB).
    assert "172.22" in listing.strip().splitlines()[-1], listing.strip().splitlines()[-1]


def test_a_small_product_over_a_moderate_k_is_one_launch_with_k_split_inside_the_workgroups():
    w = workloads.matmul_epilogue(_env(), 1000, 128, 784, upload=False)
    fused = hip_backend.check_schedule(w.graph, fused=True)
    assert int(fused.split()[0]) == 1 and "k split over the 8 waves of a workgroup" in fused and "+epilogue" in fused and "grid 256x512" in fused, fused
    # the ConvNet's first dense layer (k = 1568, two chunks in the reference's graph) the same way
    conv = hip_backend.check_schedule(workloads.convnet(_env(), batch=1000).graph, fused=True)
    assert re.search(r"MatMul \(k=1568\) \[2, 1, 1000, 128\] \+ PerElement \(7 ops\) \[128000\]  \[k split over the 8 waves", conv), conv
    # not a transposed A (a weight gradient), nor a wide output
    assert "k split over" not in hip_backend.check_schedule(workloads.matmul_epilogue(_env(), 1024, 1024, 1024, upload=False).graph, fused=True)


def test_a_row_fused_launch_runs_the_light_cluster_that_produces_its_operand():
    """hidden = leaky_relu(x . w1 + b1) is read by the classifier head's product and again by the backward pass: the
    row-fused launch that starts from the head's product evaluates the bias + activation cluster (and the sum over the
    first product's k chunks behind it) itself and stores the hidden layer on the way."""
    code = "import sys; sys.path.insert(0, %r); from descent_amd import Environment, hip_backend, workloads; from oracle.cpu_backend import CpuBackend; " \
           "print(hip_backend.check_schedule(workloads.convnet(Environment(CpuBackend()), batch=1000).graph, fused=True))"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

    def plan(**env):
        return subprocess.run([sys.executable, "-c", code % root], env=dict(os.environ, **env), check=True, capture_output=True, text=True).stdout

    # (with the first product on the kernel that splits k inside its workgroups there are no partial sums and the
    # activation is that kernel's epilogue: the fusion is looked at with that kernel switched off)
    listing = plan(DSC_MM_KSPLIT="0")
    line = next(l for l in listing.splitlines() if ": RowFused" in l)
    assert "<2 fused producers>" in line and "the first a MatMul over k=128" in line, line
    assert not any(re.match(r"\d+: PerElement \(7 ops\) \[128000\]", l) for l in listing.splitlines()), listing
    off = plan(DSC_MM_KSPLIT="0", DSC_FUSE_ROWS_OPERAND="0")
    assert int(off.split()[0]) == 9 and re.search(r"\d+: PerElement \(7 ops\) \[128000\] <1 fused producers>", off), off
    # the same launch ends with the head's data gradient, dZ x W^T masked by the hidden layer it has just stored: the
    # short-k MatMul is no launch part any more, and the gradients of the layer below share one launch with the head's
    assert "row-fused with the first stage's data gradient behind the last" in line, line
    assert "MatMul (k=10)" not in listing
    assert re.search(r"Multi \(7 kernels: .*MatMul \(k=1000\) \[13, 1, 128, 10\]; MatMul \(k=128\) \[1, 1, 1000, 1568\]; MatMul \(k=1000\) \[13, 1, 1568, 128\];\)", listing), listing
    no_tail = plan(DSC_MM_KSPLIT="0", DSC_FUSE_ROWS_DGRAD="0")
    assert int(no_tail.split()[0]) == 9 and "MatMul (k=10) [1, 1, 1000, 128]" in no_tail, no_tail


def test_the_product_a_row_fused_launch_starts_from_is_its_first_stage():
    def build(s, x, w, b, labels, loss):
        logits = _value(s, x).matmul(_value(s, w)) + _value(s, b)
        t = logits - logits.reduce_max(-1, True)
        e = t.exp()
        p = e / e.reduce_sum(-1, True)
        s.write_parameter_value(loss, (p * _value(s, labels)).reduce_sum(-1, True))

    unfused, fused = _listings([[1000, 128], [128, 10], [10], [1000, 10], [1000, 1]], build)
    assert "MatMul (k=128) [1, 1, 1000, 10]" in unfused and int(unfused.split()[0]) >= 4
    assert int(fused.split()[0]) == 1, fused
    assert "the first a MatMul over k=128 shared by the row's lanes" in fused, fused
    # a product too large for that (B would not fit a few KB of LDS per workgroup) keeps its own launch
    _, big = _listings([[1000, 2048], [2048, 10], [10], [1000, 10], [1000, 1]], build)
    assert int(big.split()[0]) >= 2 and "the first a MatMul" not in big, big


def test_scatter_adds_into_one_accumulator_share_a_launch_and_small_launches_are_grouped():
    w = workloads.hash_grid_fit(_env(), batch=1 << 12)
    listing = hip_backend.check_schedule(w.graph, fused=True)
    chains = [line for line in listing.splitlines() if "Multi (4 kernels: ScatterAdd" in line]
    assert len(chains) == 16  # one per level: the four corner updates of a level add into one table gradient
    assert all(line.count("scatter_add: global_atomic_add_f32") == 4 for line in chains)
    # the sixteen zero fills of the table gradients: one launch ahead of the steps
    assert "prefill: Multi (16 kernels: Fill(0x00000000)" in listing
    # Adam updates of the sixteen tables and the MLP: a few shared launches, not one each
    assert int(listing.split()[0]) <= 40 and len(w.graph.clusters_sorted) > 200


def test_clusters_over_small_inputs_are_evaluated_by_their_readers():
    # the float -> integer conversion of an index array of 128 KiB, read by two ScatterAdds of a megabyte of values each
    def build(s, idx, v0, v1, acc):
        i = _value(s, idx).into_u32()
        z = s.literal(0.0).value().broadcast([100000, 2])
        s.write_parameter_value(acc, z.scatter_add(_value(s, v0), -2, i).scatter_add(_value(s, v1), -2, i))

    env = _env()
    params = [env.static_parameter(sh, f"p{i}") for i, sh in enumerate([[131072], [131072, 2], [131072, 2], [100000, 2]])]
    graph = env.build_graph(lambda scope: build(scope, *params))
    unfused = hip_backend.check_schedule(graph, fused=False)
    fused = hip_backend.check_schedule(graph, fused=True)
    assert any(line.split(": ")[1].startswith("PerElement") for line in unfused.splitlines()[1:] if re.match(r"\d+: ", line))
    launches = [line for line in fused.splitlines() if re.match(r"(\d+|prefill): ", line)]
    assert not any(line.split(": ")[1].startswith("PerElement") for line in launches), fused
    assert any("ScatterAdd" in line for line in launches)
    covered = {int(c) for line in launches if " clusters " in line for c in line.split(" clusters ")[1].split()}
    assert covered == set(range(len(graph.clusters_sorted)))


def test_a_chain_of_concats_runs_a_thread_per_row_with_the_column_a_constant():
    def build(s, a, b, c, d, out):
        s.write_parameter_value(out, (_value(s, a) * 2.0).concat(_value(s, b), -1).concat(_value(s, c) + 1.0, -1).concat(_value(s, d), -1))

    unfused, fused = _listings([[65536, 2], [65536, 3], [65536, 2], [65536, 5], [65536, 12]], build)
    assert int(unfused.split()[0]) >= 3
    assert int(fused.split()[0]) == 1, fused
    assert "a thread per row of 12 columns, the column a constant of each evaluation" in fused, fused
    # the generated kernel loads each input once per row element and selects nothing at run time
    env = _env()
    params = [env.static_parameter(sh, f"q{i}") for i, sh in enumerate([[65536, 2], [65536, 3], [65536, 2], [65536, 5], [65536, 12]])]
    graph = env.build_graph(lambda sc: build(sc, *params))
    assert len(graph.clusters_sorted) >= 3


def test_full_size_hash_grid_chains_are_binned_grouped_and_read_a_slice_major_gradient():
    w = workloads.hash_grid_fit(_env(), batch=1 << 18)
    listing = hip_backend.check_schedule(w.graph, fused=True)
    lines = listing.splitlines()
    # the gradient of the sixteen concatenated two-feature encodings is read two columns at a time by 64 links:
    # its MatMul stores it slice by slice
    assert sum("product stored as 16 column slices of width 2" in line for line in lines) == 1, listing
    # accumulators of up to 8192 floats keep a copy per workgroup in LDS; the five such chains share one launch
    lds = [line for line in lines if "5 chains in one launch" in line]
    assert len(lds) == 1 and "kept in LDS per workgroup (as doubles, ds_add_f64)" in lds[0] and "grid 545x1024" in lds[0], listing
    # the eleven larger ones go through records binned by accumulator segment: all first stages in one launch, all
    # second stages in the next
    first = [i for i, line in enumerate(lines) if "11 chains in one launch, the first: scatter chain, stage 1 of 2" in line]
    second = [i for i, line in enumerate(lines) if "11 chains in one launch, the first: scatter chain, stage 2 of 2" in line]
    assert len(first) == 1 and len(second) == 1 and second[0] == first[0] + 1, listing
    assert "256 segments" in lines[first[0]] and "grid 2816x512" in lines[first[0]] and "grid 2816x1024" in lines[second[0]]
    assert int(listing.split()[0]) <= 17
    # the cluster that turns a point's two coordinates into a cell and a fraction per level (85 ops, 32 outputs of five
    # ops each) is evaluated by its readers: none of its 2 MB arrays is stored
    assert "PerElement (85 ops)" not in listing and not any("[524288]" in line for line in lines), listing
    # the whole encoding (corner indices, weights, gathers, the chain of fifteen concats) is the one launch after the
    # target image's
    assert sum("a thread per row of 32 columns" in line for line in lines) == 1, listing
    # every reference cluster is still covered
    covered = {int(c) for line in lines if " clusters " in line for c in line.split(" clusters ")[1].split()}
    assert covered == set(range(len(w.graph.clusters_sorted)))


def test_chain_switches_fall_back_to_one_launch_per_chain():
    # the switches are read once per process, so the other settings are listed by a child process
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); from descent_amd import Environment, hip_backend, workloads; "
            "from oracle.cpu_backend import CpuBackend; "
            "print(hip_backend.check_schedule(workloads.hash_grid_fit(Environment(CpuBackend()), batch=1 << 18).graph, fused=True))")
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, DSC_SCATTER_BINNED="0", DSC_CHAIN_GROUPS="0", DSC_SLICE_MAJOR="0")
    listing = subprocess.run([sys.executable, "-c", code % root], env=env, check=True, capture_output=True, text=True).stdout
    assert "chains in one launch" not in listing and "stage 1 of 2" not in listing and "column slices" not in listing
    assert listing.count("kept in LDS per workgroup") == 6      # accumulators of up to 18432 floats
    assert listing.count("scatter_add: global_atomic_add_f32 | scatter_add: global_atomic_add_f32") >= 10


def test_the_sign_of_a_pre_activation_is_read_off_the_stored_activation():
    graph = workloads.convnet(_env(), batch=1000).graph
    fused = hip_backend.check_schedule(graph, fused=True)
    lines = [l for l in fused.splitlines() if re.match(r"\d+: ", l)]

    def moved(line):
        return float(re.search(r"grid \S+ ([0-9.]+) MB", line).group(1))

    # The reference's convolution clusters store z = conv + bias beside a = leaky_relu(z), and the backward pass reads
    # z again for "(z > 0) ? g : 0.01 g".  a has the sign of z, so the readers test a > 0 and z is never written:
    # conv1's kernel writes a (50.2 MB) and the pooled a (12.5 MB) for its 3.1 MB image, conv2's a (25.1), the pooled
    # and dropped-out a (2 x 6.3) for 12.5 MB in
    # (and a itself gives way to two bits per element once the pooling gradients read those: 15.7 MB out for conv1,
    # 7.8 MB for conv2, whose pooled a was kept for the pooling gradient alone)
    assert "ConvForward" in lines[0] and 18.0 < moved(lines[0]) < 19.5, lines[0]     # 116.0 with z stored, 65.9 with a stored
    assert lines[1].split(": ")[1].startswith("ConvForward") and 20.0 < moved(lines[1]) < 21.0, lines[1]  # 75.3 with z stored, 50.2 with a stored
    assert "172.22" in fused.splitlines()[-1], fused.splitlines()[-1]  # MB per step; 565 with z stored, 414 before conv2's dC became a producer, 358 with fc1's k chunks in memory, 338.4 with the activations stored for the pooling gradients, 178.5 with conv2's pooled array stored
    # cluster by cluster nothing is rewritten
    unfused = hip_backend.check_schedule(graph, fused=False)
    assert "PerElement (7 ops) [12544000]" in unfused and "2316." in unfused.splitlines()[-1], unfused.splitlines()[-1]


def test_data_and_weight_gradient_of_a_layer_with_few_outputs_share_one_pass_over_the_activation():
    def build(masked_by_x):
        def fn(s, dy, x, w, other, dz, dw):
            d, xv = _value(s, dy), _value(s, x)
            p = d.matmul(_value(s, w).transpose())
            mask = xv if masked_by_x else _value(s, other)
            s.write_parameter_value(dz, mask.select_gt(0.0, p, p * 0.01))
            s.write_parameter_value(dw, xv.transpose().matmul(d))
        return fn

    shapes = [[65536, 2], [65536, 128], [128, 2], [65536, 128], [65536, 128], [128, 2]]
    unfused, fused = _listings(shapes, build(True))
    # cluster by cluster: a short-k product, its consumer, the product over the rows in the reference's 1024-deep chunks
    # and the sum of those
    assert "short-k fma" in unfused and "chunks 64" in unfused and int(unfused.split()[0]) == 5
    # fused: the weight gradient's 256 chunks are the row chunks of the data gradient's kernel; their sum is untouched
    assert int(fused.split()[0]) == 2
    assert "+the weight gradient X^T A over 256 chunks of 256 rows" in fused and "tall-k" not in fused
    assert re.search(r"Reduce \(k=256\) \[1, 1, 128, 2\]", fused)
    # a consumer that does not read the activation gains nothing from the pairing: both products stay as they are
    _, apart = _listings(shapes, build(False))
    assert "+the weight gradient" not in apart and "tall-k mfma 16x16x4" in apart


def test_surplus_k_chunks_keep_the_bounds_checked_register_path():
    """A MatMul descriptor may name more k chunks than k has tiles for (k = 64 in 3 chunks of 32: the third starts at
    k).  The tiles-straight-into-LDS path does not clamp k, so such a product must not take it; the same product with
    chunks that cover k exactly does."""
    from descent_amd import kernel as K
    from descent_amd.shape import BATCHES, Shape

    def direct(chunks, k):
        kern = K.MatMulKernel(Shape((chunks, 1, 256, 256)), BATCHES, Shape((1, 256, k)).identity_view(), Shape((1, k, 256)).identity_view())
        return int(re.search(r"#define MM_DIRECT (\d+)", hip_backend.codegen_source(kern)).group(1))

    assert direct(2, 64) > 0
    assert direct(3, 64) == 0
    assert direct(3, 96) > 0
    assert direct(5, 128) == 0  # chunks of 32: 5 * 32 > 128


def test_masked_data_gradients_read_the_sign_bytes_the_forward_products_write():
    """cfg4: the three hidden layers whose data gradient is needed are masked by (a > 0) of the stored activation; the
    forward products that write those activations add a byte per four elements, the gradients read the bytes."""
    code = "import sys; sys.path.insert(0, %r); from descent_amd import Environment, hip_backend, workloads; from oracle.cpu_backend import CpuBackend; " \
           "print(hip_backend.check_schedule(workloads.coordinate_mlp(Environment(CpuBackend())).graph, fused=True))"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

    def plan(**env):
        return subprocess.run([sys.executable, "-c", code % root], env=dict(os.environ, **env), check=True, capture_output=True, text=True).stdout

    on, off = plan(), plan(DSC_SIGN_BYTES="0")
    assert on.count("masks by sign bytes") == 3 and on.count("writes its output's sign bytes") == 3, on
    assert "sign bytes" not in off
    # 3 x 268 MB of activations not read again, 3 x 16.8 MB of bytes written and read
    assert "7318.3" in on.strip().splitlines()[-1] and "8022.9" in off.strip().splitlines()[-1], (on.strip().splitlines()[-1], off.strip().splitlines()[-1])


def test_the_backward_of_a_strided_depthwise_convolution_is_one_launch_of_gathered_sums(monkeypatch):
    """The blur of a MaxBlurPool2D (src/module.rs:219-246: 3x3, stride 2, a group per channel) leaves, in the backward
    pass, MatMul(k=1) -> copy -> WindowsToImage -> Unpad -> Unpad (src/array.rs:954-975,989-1031).  One launch evaluates
    the chain per element of the last Unpad; the gradient of the stride-1 max pooling behind it, which would evaluate it
    once per window, reads it from memory.  The forward product of one column per channel runs with its lanes along
    the channels."""
    env = _env()
    w = workloads.convnet(env, batch=16, seed=1, blur_pool=True)
    fused = hip_backend.check_schedule(w.graph, fused=True)
    assert fused.count("lanes along the batches of a row") == 2, fused
    assert "MatMul (k=1)" not in fused and fused.count("Unpad [") == 2 and fused.count("WindowsToImage [") == 2, fused
    for line in fused.splitlines():
        if "Unpad [" in line:
            # the chain behind each remaining Unpad: its producers' clusters are covered by its launch
            assert len(re.search(r"clusters ([\d ]+)$", line).group(1).split()) >= 5, line
    monkeypatch.setenv("DSC_FUSE_GATHER_SUMS", "0")
    apart = hip_backend.check_schedule(workloads.convnet(_env(), batch=16, seed=1, blur_pool=True).graph, fused=True)
    assert apart.count("Unpad [") == 4 and apart.count("MatMul (k=1)") == 2 and int(apart.split()[0]) > int(fused.split()[0])


def test_a_row_fused_launch_takes_the_light_producer_in_front_of_it(monkeypatch):
    """The linear classifier's logits are the sum of a product's ten k-chunks with the bias on it (a per-element
    cluster over a short Reduce), read element for element by the stages of the softmax cross-entropy
    (src/loss.rs:4-34): the row-fused launch evaluates it, 5 -> 4 launches."""
    w = workloads.linear_classifier(_env(), batch=1000, seed=1)
    fused = hip_backend.check_schedule(w.graph, fused=True)
    assert int(fused.split()[0]) == 4, fused
    assert re.search(r"RowFused \[1000, 10\] \(\d+ clusters\) <2 fused producers>", fused), fused
    monkeypatch.setenv("DSC_ROWS_TAKE_PRODUCERS", "0")
    apart = hip_backend.check_schedule(workloads.linear_classifier(_env(), batch=1000, seed=1).graph, fused=True)
    assert int(apart.split()[0]) == 5 and "PerElement (3 ops) [10000] <1 fused producers>" in apart, apart
