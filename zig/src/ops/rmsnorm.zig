//! RMSNorm over the last dimension with a gain vector, as an op module (not compiled in this
//! repository).
//!
//!   forward   r_i = 1 / sqrt(mean_j x[i, j]^2 + eps),   z[i, j] = x[i, j] * r_i * g[j]
//!   reverse   c_i = mean_j(z.grad[i, j] * g[j] * x[i, j])
//!             x.grad[i, j] += r_i * (z.grad[i, j] * g[j] - x[i, j] * r_i^2 * c_i)
//!             g.grad[j]    += sum_i z.grad[i, j] * x[i, j] * r_i
//!
//! x is taken as [m, n] with n its last size and g has n elements. The reverse is two kernels
//! behind one launcher: the row pass, which leaves one partial row of gain-gradient sums per
//! workgroup in the workspace, and a fixed-order sum of those rows, so g.grad does not depend on
//! scheduling. The workspace comes from the stream's scratch (src/core/utils.zig:20-36) and is
//! sized by mpRmsnormReverseScratchBytes; whether the forward wants one is for mpRmsnormScratchBytes to say
//! (0 for rows that one workgroup holds).
const std = @import("std");
const core = @import("core");
const OpDatum = core.OpDatum;
const Tensor = core.Tensor;
const Graph = core.Graph;
const dev = core.utils.dev;

fn last_size(t: Tensor) usize {
    const s = t.sizes();
    std.debug.assert(s.len >= 1);
    return s[s.len - 1];
}

pub fn forward(x: Tensor, gain: Tensor, eps: f64) Tensor {
    return forward_impl(x.ptr, x, gain, eps);
}

pub fn forward_impl(graph: *Graph, x: Tensor, gain: Tensor, eps: f64) Tensor {
    const n = last_size(x);
    std.debug.assert(gain.len() == n);
    std.debug.assert(gain.dtype() == x.dtype());
    const m = if (n == 0) 0 else x.len() / n;

    const out = graph.tensor(.{ .class = .hid, .dtype = x.dtype(), .sizes = x.sizes() });
    const key = core.dkey(out);

    const bytes = dev.mpRmsnormScratchBytes(key, m, n);
    const scratch: ?*anyopaque = if (bytes > 0) out.stream().get_scratch(.r32, (bytes + 3) / 4) else null;
    core.invoke(core.kernels.rmsnorm_ij_j, key, .{
        x.data_ptr(), gain.data_ptr(), out.data_ptr(), scratch, eps, m, n, out.context(),
    });

    if (graph.mode == .train) {
        core.attach_op(@This(), out, &.{
            OpDatum{ .tensor = x },
            OpDatum{ .tensor = gain },
            OpDatum{ .scalar = eps },
            OpDatum{ .tensor = out },
        });
    }
    return out;
}

pub fn reverse(args: []const OpDatum) void {
    const x = args[0].tensor;
    const gain = args[1].tensor;
    const eps = args[2].scalar;
    const out = args[3].tensor;
    core.enable_gradient(x);
    core.enable_gradient(gain);

    const n = last_size(x);
    const m = if (n == 0) 0 else x.len() / n;
    const key = core.dkey(out);

    // never zero bytes for a non-empty problem: the partial gain rows always go through it
    const bytes = dev.mpRmsnormReverseScratchBytes(key, m, n);
    const scratch = out.stream().get_scratch(.r32, (bytes + 3) / 4);
    core.invoke(core.kernels.rmsnorm_ij_j_reverse, key, .{
        x.data_ptr(), gain.data_ptr(), out.grad_ptr(), x.grad_ptr(), gain.grad_ptr(), scratch,
        eps, @as(f64, 1.0), m, n, out.context(),
    });
}

pub fn derive(_: []const OpDatum, _: Tensor) ?OpDatum {
    return null;
}
