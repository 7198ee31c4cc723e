//! `src/kernel_marshal.rs` -- turns the crate's kernel descriptors into the POD descriptors of the C ABI.
//!
//! `GenericKernel` (src/kernel.rs:878-886) and everything it holds (`View`, `Shape`, `PerElementKernelOp`) stay as they
//! are; the GLSL text generators (`Kernel::generate_source`, src/kernel.rs:135-874) are no longer called.  A kernel is
//! described to the library by value -- the library's cache is keyed by the descriptor's content exactly as
//! `KernelCache::module` is keyed by `#[derive(Hash, Eq)]` (src/kernel.rs:1037-1056) -- and a whole `Graph`
//! (src/graph.rs:102-108) is handed over once as a `dsc_schedule_desc`, which is what lets the library fuse across
//! clusters.
//!
//! The arrays a descriptor points into live in the `Marshalled*` value that produced it; keep that value alive for
//! as long as the raw descriptor is in use (the library deep-copies on `dsc_kernel_get` / `dsc_schedule_create`, so
//! that is only until those calls return).

use crate::common::*;
use crate::device::hip::*;
use petgraph::visit::{IntoNodeReferences, NodeRef};
use std::collections::HashMap;

fn c_shape(shape: &Shape) -> dsc_shape {
    let mut out = dsc_shape { rank: shape.len() as i32, dims: [0; DSC_MAX_DIM] };
    for (dst, &src) in out.dims.iter_mut().zip(shape.iter()) {
        *dst = src as i64;
    }
    out
}

fn c_shape_1d(element_count: usize) -> dsc_shape {
    let mut out = dsc_shape { rank: 1, dims: [0; DSC_MAX_DIM] };
    out.dims[0] = element_count as i64;
    out
}

/// `View` (src/shape.rs:354-360): `AxisMapping::Source { axis, step }` becomes `(map_axis, map_step)`,
/// `AxisMapping::Broadcast` becomes `map_axis = -1` (src/shape.rs:322-325).
fn c_view(view: &View) -> dsc_view {
    let mut out = dsc_view {
        in_shape: c_shape(&view.input_shape),
        in_offset: [0; DSC_MAX_DIM],
        out_shape: c_shape(&view.output_shape),
        map_axis: [-1; DSC_MAX_DIM],
        map_step: [0; DSC_MAX_DIM],
    };
    for (dst, &src) in out.in_offset.iter_mut().zip(view.input_offsets.iter()) {
        *dst = src as i64;
    }
    for (j, mapping) in view.output_mapping.iter().enumerate() {
        match *mapping {
            AxisMapping::Source { axis, step } => {
                out.map_axis[j] = axis.index() as i32;
                out.map_step[j] = step as i64;
            }
            AxisMapping::Broadcast => {
                out.map_axis[j] = -1;
                out.map_step[j] = 0;
            }
        }
    }
    out
}

fn literal_bits(value: Literal) -> u32 {
    match value {
        Literal::F32(v) => v.into_inner().to_bits(),
        Literal::U32(v) => v,
    }
}

fn unary_code(op: UnaryOp) -> i32 {
    // dsc_unary_op lists the variants in the order of src/op.rs:59-70
    match op {
        UnaryOp::Mov => 0,
        UnaryOp::Neg => 1,
        UnaryOp::Sqrt => 2,
        UnaryOp::Exp => 3,
        UnaryOp::Log => 4,
        UnaryOp::Sin => 5,
        UnaryOp::Cos => 6,
        UnaryOp::FloatToUint => 7,
        UnaryOp::UintToFloat => 8,
    }
}

fn binary_code(op: BinaryOp) -> i32 {
    // dsc_binary_op, src/op.rs:46-57
    match op {
        BinaryOp::Add => 0,
        BinaryOp::Sub => 1,
        BinaryOp::Mul => 2,
        BinaryOp::Div => 3,
        BinaryOp::Pow => 4,
        BinaryOp::UAdd => 5,
        BinaryOp::UMul => 6,
        BinaryOp::URem => 7,
        BinaryOp::UBitXor => 8,
    }
}

fn compare_code(mode: CompareMode) -> i32 {
    match mode {
        CompareMode::Eq => 0,
        CompareMode::Gt => 1,
    }
}

fn reduce_code(op: ReduceOp) -> i32 {
    match op {
        ReduceOp::Max => 0,
        ReduceOp::Sum => 1,
    }
}

fn output_mode_code(mode: MatMulOutputMode) -> i32 {
    match mode {
        MatMulOutputMode::Batches => 0,
        MatMulOutputMode::Rows => 1,
    }
}

/// One `GenericKernel` as a `dsc_kernel_desc` plus the arrays it points into.
pub(crate) struct MarshalledKernel {
    pub(crate) desc: dsc_kernel_desc,
    views: Vec<dsc_view>,
    ops: Vec<dsc_pe_op>,
    outputs: Vec<i32>,
    builtin_views: Vec<dsc_view>,
}

impl MarshalledKernel {
    pub(crate) fn new(kernel: &GenericKernel) -> Box<Self> {
        let mut desc = dsc_kernel_desc {
            kind: 0,
            shape: c_shape_1d(1),
            n_inputs: 0,
            inputs: std::ptr::null(),
            n_ops: 0,
            ops: std::ptr::null(),
            n_outputs: 0,
            outputs: std::ptr::null(),
            n_builtin_views: 0,
            builtin_views: std::ptr::null(),
            fill_bits: 0,
            reduce_op: 0,
            axis: 0,
            pad: 0,
            stride_w: 0,
            stride_h: 0,
            output_mode: 0,
        };
        let mut views = Vec::new();
        let mut ops = Vec::new();
        let mut outputs = Vec::new();
        let mut builtin_views = Vec::new();
        match kernel {
            GenericKernel::Fill(k) => {
                desc.kind = DSC_KERNEL_FILL;
                desc.shape = c_shape_1d(k.element_count);
                desc.fill_bits = literal_bits(k.value);
            }
            GenericKernel::PerElement(k) => {
                desc.kind = DSC_KERNEL_PER_ELEMENT;
                desc.shape = c_shape_1d(k.element_count);
                views.extend(k.inputs.iter().map(c_view));
                outputs.extend(k.outputs.iter().map(|&i| i as i32));
                for op in k.ops.iter() {
                    let mut o = dsc_pe_op {
                        kind: 0,
                        op: 0,
                        args: [0; 4],
                        bits: 0,
                        input_index: 0,
                        view_index: 0,
                        axis: 0,
                        gather_shape: c_shape_1d(1),
                    };
                    match *op {
                        PerElementKernelOp::Load { input_index } => {
                            o.kind = DSC_PE_LOAD;
                            o.input_index = input_index as i32;
                        }
                        PerElementKernelOp::Literal(value) => {
                            o.kind = match value {
                                Literal::F32(_) => DSC_PE_LITERAL_F32,
                                Literal::U32(_) => DSC_PE_LITERAL_U32,
                            };
                            o.bits = literal_bits(value);
                        }
                        PerElementKernelOp::BuiltIn { op: built_in, view } => {
                            o.view_index = builtin_views.len() as i32;
                            builtin_views.push(c_view(&view));
                            match built_in {
                                BuiltInOp::Coord => o.kind = DSC_PE_COORD,
                                BuiltInOp::Rand { uid } => {
                                    o.kind = DSC_PE_RAND;
                                    o.bits = uid as u32;
                                }
                            }
                        }
                        PerElementKernelOp::Unary { op: unary, args } => {
                            o.kind = DSC_PE_UNARY;
                            o.op = unary_code(unary);
                            o.args[0] = args as i32;
                        }
                        PerElementKernelOp::Binary { op: binary, args } => {
                            o.kind = DSC_PE_BINARY;
                            o.op = binary_code(binary);
                            o.args[0] = args[0] as i32;
                            o.args[1] = args[1] as i32;
                        }
                        PerElementKernelOp::CompareAndSelect { compare_mode, args } => {
                            o.kind = DSC_PE_SELECT;
                            o.op = compare_code(compare_mode);
                            for (dst, &src) in o.args.iter_mut().zip(args.iter()) {
                                *dst = src as i32;
                            }
                        }
                        PerElementKernelOp::Gather { shape, axis, input_index, arg } => {
                            o.kind = DSC_PE_GATHER;
                            o.input_index = input_index as i32;
                            o.axis = axis.index() as i32;
                            o.args[0] = arg as i32;
                            o.gather_shape = c_shape(&shape);
                        }
                    }
                    ops.push(o);
                }
            }
            GenericKernel::Reduce(k) => {
                desc.kind = DSC_KERNEL_REDUCE;
                desc.shape = c_shape(&k.shape);
                views.push(c_view(&k.input));
                desc.reduce_op = reduce_code(k.reduce_op);
                desc.axis = k.axis.index() as i32;
            }
            GenericKernel::MatMul(k) => {
                desc.kind = DSC_KERNEL_MATMUL;
                desc.shape = c_shape(&k.shape);
                views.push(c_view(&k.a));
                views.push(c_view(&k.b));
                desc.output_mode = output_mode_code(k.output_mode);
            }
            GenericKernel::Unpad(k) => {
                desc.kind = DSC_KERNEL_UNPAD;
                desc.shape = c_shape(&k.shape);
                views.push(c_view(&k.input));
                desc.axis = k.axis.index() as i32;
                desc.pad = k.pad as i32;
            }
            GenericKernel::WindowsToImage(k) => {
                desc.kind = DSC_KERNEL_WINDOWS_TO_IMAGE;
                desc.shape = c_shape(&k.shape);
                views.push(c_view(&k.input));
                // the tuple is (w, h): src/kernel.rs:716,740
                desc.stride_w = k.stride.0 as i32;
                desc.stride_h = k.stride.1 as i32;
            }
            GenericKernel::ScatterAdd(k) => {
                desc.kind = DSC_KERNEL_SCATTER_ADD;
                desc.shape = c_shape(&k.shape);
                views.push(c_view(&k.values));
                views.push(c_view(&k.indices));
                desc.axis = k.axis.index() as i32;
            }
        }
        // boxed so that the vectors' heap storage, not the struct, is what the raw pointers refer to: moving the box
        // does not move them
        let mut out = Box::new(Self { desc, views, ops, outputs, builtin_views });
        out.desc.n_inputs = out.views.len() as i32;
        out.desc.inputs = out.views.as_ptr();
        out.desc.n_ops = out.ops.len() as i32;
        out.desc.ops = out.ops.as_ptr();
        out.desc.n_outputs = out.outputs.len() as i32;
        out.desc.outputs = out.outputs.as_ptr();
        out.desc.n_builtin_views = out.builtin_views.len() as i32;
        out.desc.builtin_views = out.builtin_views.as_ptr();
        out
    }
}

/// A whole `Graph` as a `dsc_schedule_desc`.  `params[slot]` names the parameter behind each slot of the `params`
/// array that `dsc_schedule_run` takes.
pub(crate) struct MarshalledSchedule {
    pub(crate) desc: dsc_schedule_desc,
    pub(crate) params: Vec<ParameterId>,
    kernels: Vec<Box<MarshalledKernel>>,
    clusters: Vec<dsc_cluster>,
    cluster_inputs: Vec<Vec<i32>>,
    cluster_outputs: Vec<Vec<dsc_cluster_output>>,
    node_elements: Vec<i64>,
    inputs: Vec<dsc_param_io>,
    outputs: Vec<dsc_param_io>,
}

/// Identifies a graph by content: a hash over everything `MarshalledSchedule::new` reads (the element count of
/// every node, the parameter behind each Input / Output node, and per cluster its kernel descriptor, its input and
/// output nodes and their initial states).  Two graphs with the same fingerprint marshal to the same schedule and
/// the same parameter slots, so a schedule cached under it is valid for either.  An address of something inside the
/// `Graph` is not: a graph dropped and rebuilt (per epoch, in a loop) can put its vectors where the old one's were.
/// The reference pays the same kind of cost per run: one `HashMap<GenericKernel, _>` lookup per cluster
/// (src/kernel.rs:1050).
pub(crate) fn graph_fingerprint(graph: &Graph) -> u64 {
    use std::hash::{Hash, Hasher};
    let mut h = std::collections::hash_map::DefaultHasher::new();
    graph.ops.node_bound().hash(&mut h);
    for node_ref in graph.ops.node_references() {
        let node_id = node_ref.id();
        node_id.index().hash(&mut h);
        node_ref.weight().shape.element_count().hash(&mut h);
        match node_ref.weight().op {
            Op::Input { parameter_id } => (1u8, parameter_id).hash(&mut h),
            Op::Output { parameter_id } => {
                (2u8, parameter_id).hash(&mut h);
                for source in get_arg_sources(&graph.ops, node_id).iter() {
                    source.node_id.index().hash(&mut h);
                }
            }
            _ => 0u8.hash(&mut h),
        }
    }
    graph.clusters_sorted.len().hash(&mut h);
    for cluster_id in graph.clusters_sorted.iter().copied() {
        let cluster = &graph.clusters[cluster_id];
        cluster.kernel.hash(&mut h);
        cluster.inputs.len().hash(&mut h);
        for n in cluster.inputs.iter() {
            n.index().hash(&mut h);
        }
        cluster.outputs.len().hash(&mut h);
        for output in cluster.outputs.iter() {
            output.node_id.index().hash(&mut h);
            match output.initial_state {
                InitialState::CopyFrom(src_node_id) => {
                    (1u8, src_node_id.index()).hash(&mut h);
                    if let Op::Literal(value) = graph.ops[src_node_id].op {
                        literal_bits(value).hash(&mut h);
                    }
                }
                _ => 0u8.hash(&mut h),
            }
        }
    }
    h.finish()
}

impl MarshalledSchedule {
    pub(crate) fn new(graph: &Graph) -> Box<Self> {
        let mut params: Vec<ParameterId> = Vec::new();
        let mut slot_of: HashMap<ParameterId, i32> = HashMap::new();
        let mut slot = |id: ParameterId, params: &mut Vec<ParameterId>| -> i32 {
            *slot_of.entry(id).or_insert_with(|| {
                params.push(id);
                (params.len() - 1) as i32
            })
        };

        let mut node_elements = vec![0i64; graph.ops.node_bound()];
        let mut inputs = Vec::new();
        let mut outputs = Vec::new();
        for node_ref in graph.ops.node_references() {
            let node_id = node_ref.id();
            node_elements[node_id.index()] = node_ref.weight().shape.element_count() as i64;
            match node_ref.weight().op {
                // src/environment.rs:330-340
                Op::Input { parameter_id } => inputs.push(dsc_param_io {
                    node: node_id.index() as i32,
                    param: slot(parameter_id, &mut params),
                }),
                // src/environment.rs:341-351, 506-515: the parameter takes the buffer of the Output node's only source
                Op::Output { parameter_id } => {
                    let arg_sources = get_arg_sources(&graph.ops, node_id);
                    assert_eq!(arg_sources.len(), 1);
                    outputs.push(dsc_param_io {
                        node: arg_sources[0].node_id.index() as i32,
                        param: slot(parameter_id, &mut params),
                    });
                }
                _ => {}
            }
        }

        let mut kernels = Vec::new();
        let mut cluster_inputs = Vec::new();
        let mut cluster_outputs = Vec::new();
        for cluster_id in graph.clusters_sorted.iter().copied() {
            let cluster = &graph.clusters[cluster_id];
            kernels.push(MarshalledKernel::new(&cluster.kernel));
            cluster_inputs.push(cluster.inputs.iter().map(|n| n.index() as i32).collect::<Vec<_>>());
            cluster_outputs.push(
                cluster
                    .outputs
                    .iter()
                    .map(|output| {
                        let mut out = dsc_cluster_output {
                            node: output.node_id.index() as i32,
                            copy_from: -1,
                            copy_from_is_literal: 0,
                            literal_bits: 0,
                        };
                        // src/environment.rs:407-444: CopyFrom takes the source's buffer over, or starts from a Fill
                        // when the source is a literal
                        if let InitialState::CopyFrom(src_node_id) = output.initial_state {
                            out.copy_from = src_node_id.index() as i32;
                            if let Op::Literal(value) = graph.ops[src_node_id].op {
                                out.copy_from_is_literal = 1;
                                out.literal_bits = literal_bits(value);
                            }
                        }
                        out
                    })
                    .collect::<Vec<_>>(),
            );
        }
        let clusters = kernels
            .iter()
            .zip(cluster_inputs.iter())
            .zip(cluster_outputs.iter())
            .map(|((kernel, ins), outs)| dsc_cluster {
                kernel: kernel.desc,
                n_inputs: ins.len() as i32,
                inputs: ins.as_ptr(),
                n_outputs: outs.len() as i32,
                outputs: outs.as_ptr(),
            })
            .collect::<Vec<_>>();

        let mut out = Box::new(Self {
            desc: dsc_schedule_desc {
                n_nodes: 0,
                node_elements: std::ptr::null(),
                n_clusters: 0,
                clusters: std::ptr::null(),
                n_inputs: 0,
                inputs: std::ptr::null(),
                n_outputs: 0,
                outputs: std::ptr::null(),
                n_params: 0,
            },
            params,
            kernels,
            clusters,
            cluster_inputs,
            cluster_outputs,
            node_elements,
            inputs,
            outputs,
        });
        out.desc.n_nodes = out.node_elements.len() as i32;
        out.desc.node_elements = out.node_elements.as_ptr();
        out.desc.n_clusters = out.clusters.len() as i32;
        out.desc.clusters = out.clusters.as_ptr();
        out.desc.n_inputs = out.inputs.len() as i32;
        out.desc.inputs = out.inputs.as_ptr();
        out.desc.n_outputs = out.outputs.len() as i32;
        out.desc.outputs = out.outputs.as_ptr();
        out.desc.n_params = out.params.len() as i32;
        out
    }
}
