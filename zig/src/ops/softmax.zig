//! Softmax over the last dimension as an op module (not compiled in this repository).
//!
//!   forward   z[i, :] = exp(x[i, :] - max_j x[i, j]) / sum_j exp(x[i, j] - max_j x[i, j])
//!   reverse   x.grad[i, j] += z[i, j] * (z.grad[i, j] - sum_k z[i, k] * z.grad[i, k])
//!
//! A tensor of any rank is taken as [m, n] with n its last size, the way the reference's row
//! reductions take theirs (src/ops/reduce.zig:98-121). The reverse needs the forward OUTPUT, so
//! the op keeps (x, z) like every unary op. Long rows are shared by several workgroups through a
//! workspace from the stream's scratch (src/core/utils.zig:20-36), which the reference's own
//! softmax call sites already pass (src/loss/loss.zig:204,226); the size functions say how much
//! (0 for rows of up to 32 KiB, and then no workspace is taken at all).
const std = @import("std");
const core = @import("core");
const OpDatum = core.OpDatum;
const Tensor = core.Tensor;
const Graph = core.Graph;
const dev = core.utils.dev;

const Rows = struct { m: usize, n: usize };

fn rows_of(t: Tensor) Rows {
    const s = t.sizes();
    std.debug.assert(s.len >= 1);
    const n = s[s.len - 1];
    return .{ .m = if (n == 0) 0 else t.len() / n, .n = n };
}

/// `bytes` of the stream's scratch as whole r32 words, or null when the launcher wants none.
fn workspace(t: Tensor, bytes: usize) ?*anyopaque {
    if (bytes == 0) return null;
    return t.stream().get_scratch(.r32, (bytes + 3) / 4);
}

pub fn forward(x: Tensor) Tensor {
    return forward_impl(x.ptr, x);
}

pub fn forward_impl(graph: *Graph, x: Tensor) Tensor {
    const out = graph.tensor(.{ .class = .hid, .dtype = x.dtype(), .sizes = x.sizes() });
    const key = core.dkey(out);
    const r = rows_of(x);

    const scratch = workspace(out, dev.mpSoftmaxScratchBytes(key, r.m, r.n));
    core.invoke(core.kernels.softmax_ij_j, key, .{ x.data_ptr(), out.data_ptr(), scratch, r.m, r.n, out.context() });

    if (graph.mode == .train) {
        core.attach_op(@This(), out, &.{ OpDatum{ .tensor = x }, OpDatum{ .tensor = out } });
    }
    return out;
}

pub fn reverse(args: []const OpDatum) void {
    const x = args[0].tensor;
    const out = args[1].tensor;
    core.enable_gradient(x);
    const key = core.dkey(out);
    const r = rows_of(out);

    const scratch = workspace(out, dev.mpSoftmaxReverseScratchBytes(key, r.m, r.n));
    // alpha = 1: dst = val + alpha * dst, the blend of src/cuda/nvcc_src/reduce_ij_i.cu:31
    core.invoke(core.kernels.softmax_ij_j_reverse, key, .{
        out.data_ptr(), out.grad_ptr(), x.grad_ptr(), scratch, @as(f64, 1.0), r.m, r.n, out.context(),
    });
}

pub fn derive(_: []const OpDatum, _: Tensor) ?OpDatum {
    return null;
}
