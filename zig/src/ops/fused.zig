//! Elementwise ops that are recorded instead of launched, so that a whole pending expression runs
//! as one kernel per direction (not compiled in this repository: no Zig toolchain there).
//!
//! The reference launches every elementwise op by itself, through a temporary of its own
//! (src/ops/addition.zig:27-58, src/ops/hadamard.zig:25-56). With this layer on
//! (`mp.ops.fusion.enable()`), `add`, `hadamard`, `selu` and the others call `record` instead: the
//! result tensor exists (its storage comes from graph.tensor as always) but nothing is enqueued.
//! The first time its bytes or its op are needed -- Tensor.data_ptr() and Tensor.reverse() call the
//! hook this module installs in src/core/graph.zig -- the pending expression below it is spelled
//! with its leaves numbered in order of first appearance ("selu(mul(add(0,1),add(2,3)))"), and
//!   * an expression the build listed (fused_chains.zig, written by the kernel generator from
//!     chains.json) runs as its launch_fused_* launcher: ONE kernel, and ONE reverse kernel that
//!     writes every leaf gradient;
//!   * any other expression of two or more ops goes to mpChainForward / mpChainReverse, which
//!     compile it on first use (lib/libmp_fusion.so; the constants of dilate and translate are
//!     kernel arguments, so a value that changes from call to call compiles nothing);
//!   * a single op, or a refusal of the fusion library, runs op by op as the reference does.
//! Pending nodes inside a fused expression are never computed: their gradients do not exist.
//! Code that wants them (the reference's examples assert the gradients of intermediates)
//! leaves the layer off, which is the default.
const std = @import("std");
const core = @import("core");
const OpDatum = core.OpDatum;
const Tensor = core.Tensor;
const Graph = core.Graph;
const StreamContext = core.utils.StreamContext;
const chains = @import("fused_chains.zig");

// include/chain_fusion.h
extern fn mpChainForward(expression: [*:0]const u8, dtype: c_int, x: [*]const ?*const anyopaque, out: ?*anyopaque, n: c_ulong, ctx: StreamContext) c_int;
extern fn mpChainReverse(expression: [*:0]const u8, dtype: c_int, x: [*]const ?*const anyopaque, out_grads: ?*const anyopaque, g: [*]const ?*anyopaque, alpha: f64, n: c_ulong, ctx: StreamContext) c_int;
extern fn mpChainCompile(expression: [*:0]const u8, dtype: c_int) c_int;
extern fn mpChainError() [*:0]const u8;

pub const Op = enum { add, sub, mul, selu, relu, scale, shift };

const max_leaves = 8;
const max_nodes = 64;

const Node = struct { op: Op, in0: Tensor, in1: ?Tensor, value: f64 };
const Key = struct { graph: usize, idx: usize };

pub var enabled: bool = false;
var pending: std.AutoHashMapUnmanaged(Key, Node) = .{};
const allocator = std.heap.c_allocator;

pub fn enable() void {
    core.cg.materialise_hook = &materialise;
    core.cg.forget_hook = &forget;
    enabled = true;
}

/// Computes what is still pending when asked for it, then stops recording.
pub fn disable() void {
    enabled = false;
}

/// The hook of Graph.reset(.node, .all): what was recorded against the nodes of a graph goes
/// with them (their indices start over).
fn forget(g: *Graph) void {
    var stale = std.ArrayListUnmanaged(Key){};
    defer stale.deinit(allocator);
    var it = pending.keyIterator();
    while (it.next()) |k| {
        if (k.graph == @intFromPtr(g)) stale.append(allocator, k.*) catch @panic("fused: out of memory");
    }
    for (stale.items) |k| _ = pending.remove(k);
}

fn key_of(t: Tensor) Key {
    return .{ .graph = @intFromPtr(t.ptr), .idx = t.idx };
}

pub fn is_pending(t: Tensor) bool {
    return t.class == .hid and pending.contains(key_of(t));
}

/// What an op module's forward_impl calls instead of launching: z = op(x, y) (y null for the
/// one-operand ops, value the constant of scale / shift).
pub fn record(graph: *Graph, op: Op, x: Tensor, y: ?Tensor, value: f64) Tensor {
    const z = graph.tensor(.{ .class = .hid, .dtype = x.dtype(), .sizes = x.sizes() });
    pending.put(allocator, key_of(z), .{ .op = op, .in0 = x, .in1 = y, .value = value }) catch @panic("fused: out of memory");
    return z;
}

fn op_name(op: Op) []const u8 {
    return switch (op) {
        .add => "add",
        .sub => "sub",
        .mul => "mul",
        .selu => "selu",
        .relu => "relu",
        .scale => "scale",
        .shift => "shift",
    };
}

const Spelling = struct {
    text: std.ArrayListUnmanaged(u8) = .{},
    leaves: std.BoundedArray(Tensor, max_leaves) = .{},
    nodes: usize = 0,
    ops: usize = 0,
};

/// The expression below t as the chain table spells it: pending nodes of t's graph become
/// op(...), everything else a leaf numbered in order of first appearance (the same tensor keeps
/// its number). False beyond eight leaves or 64 nodes.
fn spell(g: *Graph, t: Tensor, s: *Spelling) bool {
    s.nodes += 1;
    if (s.nodes > max_nodes) return false;
    if (t.ptr == g) {
        if (pending.get(key_of(t))) |node| {
            s.ops += 1;
            s.text.appendSlice(allocator, op_name(node.op)) catch return false;
            s.text.append(allocator, '(') catch return false;
            if (!spell(g, node.in0, s)) return false;
            if (node.op == .scale or node.op == .shift) {
                var buf: [40]u8 = undefined;
                const lit = std.fmt.bufPrint(&buf, ",{e}", .{node.value}) catch return false;
                s.text.appendSlice(allocator, lit) catch return false;
            } else if (node.in1) |y| {
                s.text.append(allocator, ',') catch return false;
                if (!spell(g, y, s)) return false;
            }
            s.text.append(allocator, ')') catch return false;
            return true;
        }
    }
    var k: usize = 0;
    while (k < s.leaves.len and !s.leaves.get(k).same(t)) k += 1;
    if (k == s.leaves.len) s.leaves.append(t) catch return false;
    var buf: [8]u8 = undefined;
    const num = std.fmt.bufPrint(&buf, "{d}", .{k}) catch return false;
    s.text.appendSlice(allocator, num) catch return false;
    return true;
}

fn find_chain(signature: []const u8) ?usize {
    for (chains.table, 0..) |c, i| {
        if (std.mem.eql(u8, c.signature, signature)) return i;
    }
    return null;
}

/// The hook of Tensor.data_ptr() and Tensor.reverse(): a result that is still pending is computed
/// now, with everything pending below it, as one kernel where one can be had.
pub fn materialise(t: Tensor) void {
    if (t.class != .hid) return;
    const node = pending.get(key_of(t)) orelse return;
    const g = t.ptr;

    var s = Spelling{};
    defer s.text.deinit(allocator);
    const spelled = spell(g, t, &s);
    _ = pending.remove(key_of(t)); // from here on t.data_ptr() is its storage, not a call back into this function

    if (spelled) {
        const key = core.dkey(t);
        var x: [max_leaves]*anyopaque = undefined;
        for (s.leaves.slice(), 0..) |leaf, i| x[i] = leaf.data_ptr(); // a leaf that is pending in another graph is computed here
        if (find_chain(s.text.items)) |index| {
            chains.table[index].forward(key, x[0..s.leaves.len], t.data_ptr(), t.len(), t.context());
            attach(t, s.leaves.slice(), s.text.items, index);
            return;
        }
        if (s.ops >= 2) {
            s.text.append(allocator, 0) catch @panic("fused: out of memory");
            const text: [*:0]const u8 = @ptrCast(s.text.items.ptr);
            if (mpChainForward(text, @intCast(key), @ptrCast(&x), t.data_ptr(), t.len(), t.context()) == 0) {
                attach(t, s.leaves.slice(), s.text.items[0 .. s.text.items.len - 1], null);
                return;
            }
            std.log.warn("fused: {s}; running the ops one by one", .{std.mem.span(mpChainError())});
        }
    }
    one_by_one(g, t, node);
}

/// One reverse op for the whole expression: args = leaves..., the expression, the index into the
/// table (-1: compiled at run time), the result.
fn attach(t: Tensor, leaves: []const Tensor, text: []const u8, index: ?usize) void {
    if (t.ptr.mode != .train) return;
    var args = std.BoundedArray(OpDatum, max_leaves + 3){};
    for (leaves) |leaf| args.appendAssumeCapacity(.{ .tensor = leaf });
    // the text outlives this call: the graph's node arena owns the copy
    const kept = t.ptr.node_arena.allocator().dupeZ(u8, text) catch @panic("fused: out of memory");
    args.appendAssumeCapacity(.{ .expr = kept });
    args.appendAssumeCapacity(.{ .scalar = if (index) |i| @floatFromInt(i) else -1.0 });
    args.appendAssumeCapacity(.{ .tensor = t });
    core.attach_op(@This(), t, args.slice());
}

/// g[j] += d expression / d leaf j * out.grad, every j in one kernel (alpha = 1: enable_gradient
/// hands out new gradient storage zero-filled, patches/src_core_graph.zig.patch).
pub fn reverse(args: []const OpDatum) void {
    const k = args.len - 3;
    const out = args[k + 2].tensor;
    var x: [max_leaves]*anyopaque = undefined;
    var grads: [max_leaves]*anyopaque = undefined;
    for (args[0..k], 0..) |a, i| {
        core.enable_gradient(a.tensor);
        x[i] = a.tensor.data_ptr();
        grads[i] = a.tensor.grad_ptr().?;
    }
    const alpha: f64 = 1.0;
    const key = core.dkey(out);
    if (args[k + 1].scalar >= 0) {
        const index: usize = @intFromFloat(args[k + 1].scalar);
        chains.table[index].reverse(key, x[0..k], out.grad_ptr().?, grads[0..k], alpha, out.len(), out.context());
    } else {
        const text: [*:0]const u8 = @ptrCast(args[k].expr.ptr);
        if (mpChainReverse(text, @intCast(key), @ptrCast(&x), out.grad_ptr(), @ptrCast(&grads), alpha, out.len(), out.context()) != 0)
            @panic("fused: the reverse of an expression that ran forward was refused");
    }
}

/// No symbolic derivative of a fused expression: `derive` builds new forward graphs out of single
/// ops (src/ops/addition.zig:84-114), which the layer being off provides.
pub fn derive(_: []const OpDatum, _: Tensor) ?OpDatum {
    return null;
}

/// The pending node by itself, as its own op module would have run it, after its operands.
fn one_by_one(g: *Graph, t: Tensor, node: Node) void {
    const was = enabled;
    enabled = false; // the op modules launch instead of recording while this runs
    defer enabled = was;
    const x = node.in0;
    const key = core.dkey(t);
    const z = t.data_ptr();
    switch (node.op) {
        .add => core.invoke(core.kernels.addition, key, .{ x.data_ptr(), node.in1.?.data_ptr(), z, t.len(), t.context() }),
        .sub => core.invoke(core.kernels.subtraction, key, .{ x.data_ptr(), node.in1.?.data_ptr(), z, t.len(), t.context() }),
        .mul => core.invoke(core.kernels.hadamard, key, .{ x.data_ptr(), node.in1.?.data_ptr(), z, t.len(), t.context() }),
        .selu => core.invoke(core.kernels.selu, key, .{ x.data_ptr(), z, t.len(), t.context() }),
        .relu => core.invoke(core.kernels.relu, key, .{ x.data_ptr(), z, t.len(), t.context() }),
        .scale => core.invoke(core.kernels.dilate, key, .{ x.data_ptr(), node.value, z, t.len(), t.context() }),
        .shift => core.invoke(core.kernels.translate, key, .{ x.data_ptr(), node.value, z, t.len(), t.context() }),
    }
    if (g.mode != .train) return;
    switch (node.op) { // the op's own reverse, arguments in the order its module expects
        .add => core.attach_op(@import("addition.zig"), t, &.{ .{ .tensor = x }, .{ .tensor = node.in1.? }, .{ .tensor = t } }),
        .sub => core.attach_op(@import("subtraction.zig"), t, &.{ .{ .tensor = x }, .{ .tensor = node.in1.? }, .{ .tensor = t } }),
        .mul => core.attach_op(@import("hadamard.zig"), t, &.{ .{ .tensor = x }, .{ .tensor = node.in1.? }, .{ .tensor = t } }),
        .selu => core.attach_op(@import("selu.zig"), t, &.{ .{ .tensor = x }, .{ .tensor = t } }),
        .relu => core.attach_op(@import("relu.zig"), t, &.{ .{ .tensor = x }, .{ .tensor = t } }),
        .scale => core.attach_op(@import("dilate.zig"), t, &.{ .{ .tensor = x }, .{ .scalar = node.value }, .{ .tensor = t } }),
        .shift => core.attach_op(@import("translate.zig"), t, &.{ .{ .tensor = x }, .{ .scalar = node.value }, .{ .tensor = t } }),
    }
}
