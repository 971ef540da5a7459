//! SELU as an op module (not compiled in this repository: no Zig toolchain there).
//!
//!   forward   z = scale * x                      (x > 0)
//!             z = scale * alpha * (exp(x) - 1)   (x <= 0)
//!   reverse   x.grad += z.grad * (x > 0 ? scale : scale * alpha * exp(x))
//!
//! with alpha = 1.6732632, scale = 1.0507010. Same op interface as the activation the reference
//! ships (src/ops/relu.zig:9-52): `forward` for callers, `forward_impl` for the graph,
//! `reverse` for Graph.reverse. Kernels: launch_selu_* / launch_selu_reverse_*.
const std = @import("std");
const core = @import("core");
const OpDatum = core.OpDatum;
const Tensor = core.Tensor;
const Graph = core.Graph;
const fused = @import("fused.zig");

pub fn forward(x: Tensor) Tensor {
    return forward_impl(x.ptr, x);
}

pub fn forward_impl(graph: *Graph, x: Tensor) Tensor {
    // recorded, not launched: the expression it ends up in runs as one kernel (fused.zig)
    if (fused.enabled) return fused.record(graph, .selu, x, null, 0.0);

    const out = graph.tensor(.{ .class = .hid, .dtype = x.dtype(), .sizes = x.sizes() });

    core.invoke(core.kernels.selu, core.dkey(out), .{ x.data_ptr(), out.data_ptr(), out.len(), out.context() });

    if (graph.mode == .train) {
        // reverse() finds the input at 0 and the output at 1
        core.attach_op(@This(), out, &.{ OpDatum{ .tensor = x }, OpDatum{ .tensor = out } });
    }
    return out;
}

/// x.grad += out.grad * selu'(x). The launcher accumulates, as launch_relu_reverse does
/// (src/cuda/nvcc_src/relu_reverse.cu:14), so the gradient of x must exist and start at zero:
/// see patches/src_core_graph.zig.patch.
pub fn reverse(args: []const OpDatum) void {
    const x = args[0].tensor;
    const out = args[1].tensor;
    core.enable_gradient(x);
    core.invoke(core.kernels.selu_reverse, core.dkey(out), .{
        x.data_ptr(), x.grad_ptr(), out.grad_ptr(), x.len(), x.context(),
    });
}

/// No symbolic derivative: the reference's `derive` builds a new forward graph from an op's
/// derivative (src/ops/relu.zig:54-57 through stepwise.zig), and SELU's slope has no op of its own.
pub fn derive(_: []const OpDatum, _: Tensor) ?OpDatum {
    return null;
}
