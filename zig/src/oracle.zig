//! Host reference of the row-reduction / elementwise path in Zig (not compiled in this repository:
//! no Zig toolchain there). It states in fp64 the same math as oracle/mp_oracle.c, function by
//! function and loop by loop, for a box that has `zig` 0.13 and wants the host reference in the
//! reference's own language. Inputs are read in their storage type and widened to f64; every
//! output is unrounded f64. Row-major layout (src/core/tensor_components.zig:50-67).
//!
//! It is test infrastructure like its C twin: check it against tests/golden/hotpath_golden.npz
//! (written by tests/golden/make_golden.py) before trusting it, and keep it out of the op modules.
//!
//! Accumulation is f64 throughout, as the reference's `precision<T>` rule widens before it
//! reduces (src/cuda/tensor_types.h:51-69); the one-line bodies it restates are
//! src/cuda/nvcc_src/addition.cu:12, hadamard.cu:12, hadamard_reverse.cu:12, and the
//! `(a >= 0)` activation pattern of relu.cu:12 / relu_reverse.cu:14 for SELU's shape.
const std = @import("std");

pub const selu_alpha: f64 = 1.6732632;
pub const selu_scale: f64 = 1.0507010;

/// Widen one stored element. T is f16, f32 or f64 (the reference's r16, r32, r64).
inline fn wide(comptime T: type, v: T) f64 {
    return @as(f64, @floatCast(v));
}

// ---------------------------------------------------------------- elementwise

pub fn addition(comptime T: type, a: []const T, b: []const T, c: []f64) void {
    for (a, b, c) |x, y, *z| z.* = wide(T, x) + wide(T, y);
}

pub fn hadamard(comptime T: type, a: []const T, b: []const T, c: []f64) void {
    for (a, b, c) |x, y, *z| z.* = wide(T, x) * wide(T, y);
}

/// c_out = c_in + a * b (the `+=` of hadamard_reverse.cu:12).
pub fn hadamard_reverse(comptime T: type, a: []const T, b: []const T, c_in: []const T, c_out: []f64) void {
    for (a, b, c_in, c_out) |x, y, old, *z| z.* = wide(T, old) + wide(T, x) * wide(T, y);
}

pub fn selu_value(x: f64) f64 {
    return if (x > 0.0) selu_scale * x else selu_scale * selu_alpha * std.math.expm1(x);
}

pub fn selu_slope(x: f64) f64 {
    return if (x > 0.0) selu_scale else selu_scale * selu_alpha * @exp(x);
}

pub fn selu(comptime T: type, a: []const T, b: []f64) void {
    for (a, b) |x, *z| z.* = selu_value(wide(T, x));
}

/// a_grads_out = a_grads_in + b_grads * selu'(a_value); a_grads_in == null reads as zeros.
pub fn selu_reverse(comptime T: type, a_value: []const T, a_grads_in: ?[]const T, b_grads: []const T, a_grads_out: []f64) void {
    for (a_value, b_grads, a_grads_out, 0..) |x, g, *z, i| {
        const old = if (a_grads_in) |p| wide(T, p[i]) else 0.0;
        z.* = old + wide(T, g) * selu_slope(wide(T, x));
    }
}

/// e = selu((a + b) * (c + d))
pub fn fused_forward(comptime T: type, a: []const T, b: []const T, c: []const T, d: []const T, e: []f64) void {
    for (a, b, c, d, e) |av, bv, cv, dv, *z| {
        const u = wide(T, av) + wide(T, bv);
        const v = wide(T, cv) + wide(T, dv);
        z.* = selu_value(u * v);
    }
}

/// With u = a + b, v = c + d, g = de * selu'(u * v):  da = db = g * v,  dc = dd = g * u,
/// each blended as out = value + alpha * old (old == null reads as zeros).
pub fn fused_reverse(
    comptime T: type,
    a: []const T, b: []const T, c: []const T, d: []const T, de: []const T,
    old: ?[4][]const T,
    da: []f64, db: []f64, dc: []f64, dd: []f64,
    alpha: f64,
) void {
    for (a, 0..) |_, i| {
        const u = wide(T, a[i]) + wide(T, b[i]);
        const v = wide(T, c[i]) + wide(T, d[i]);
        const g = wide(T, de[i]) * selu_slope(u * v);
        const keep: [4]f64 = if (old) |o| .{
            alpha * wide(T, o[0][i]), alpha * wide(T, o[1][i]), alpha * wide(T, o[2][i]), alpha * wide(T, o[3][i]),
        } else .{ 0.0, 0.0, 0.0, 0.0 };
        da[i] = g * v + keep[0];
        db[i] = g * v + keep[1];
        dc[i] = g * u + keep[2];
        dd[i] = g * u + keep[3];
    }
}

// ---------------------------------------------------------------- softmax over the last dimension

/// y[i, j] = exp(x[i, j] - max_j) / sum_j exp(x[i, j] - max_j). An entry of -inf gives exactly 0;
/// a row without a finite entry gives NaN, as the closed form does.
pub fn softmax_ij_j(comptime T: type, x: []const T, y: []f64, m: usize, n: usize) void {
    for (0..m) |i| {
        const row = x[i * n ..][0..n];
        const out = y[i * n ..][0..n];
        var mx = -std.math.inf(f64);
        for (row) |v| mx = @max(mx, wide(T, v));
        var s: f64 = 0.0;
        for (row, out) |v, *e| {
            e.* = @exp(wide(T, v) - mx);
            s += e.*;
        }
        for (out) |*e| e.* /= s;
    }
}

/// dx[i, j] = y[i, j] * (dy[i, j] - sum_k y[i, k] * dy[i, k]) + alpha * dx_in[i, j]
pub fn softmax_ij_j_reverse(comptime T: type, y: []const T, dy: []const T, dx_in: ?[]const T, dx: []f64, alpha: f64, m: usize, n: usize) void {
    for (0..m) |i| {
        const o = i * n;
        var dot: f64 = 0.0;
        for (0..n) |j| dot += wide(T, y[o + j]) * wide(T, dy[o + j]);
        for (0..n) |j| {
            const old = if (dx_in) |p| alpha * wide(T, p[o + j]) else 0.0;
            dx[o + j] = wide(T, y[o + j]) * (wide(T, dy[o + j]) - dot) + old;
        }
    }
}

// ---------------------------------------------------------------- RMSNorm over the last dimension

/// r_i = (mean_j x[i, j]^2 + eps)^(-1/2);  y[i, j] = x[i, j] * r_i * g[j]
pub fn rmsnorm_ij_j(comptime T: type, x: []const T, g: []const T, y: []f64, eps: f64, m: usize, n: usize) void {
    const nf: f64 = @floatFromInt(n);
    for (0..m) |i| {
        const o = i * n;
        var ss: f64 = 0.0;
        for (0..n) |j| ss += wide(T, x[o + j]) * wide(T, x[o + j]);
        const r = 1.0 / @sqrt(ss / nf + eps);
        for (0..n) |j| y[o + j] = wide(T, x[o + j]) * r * wide(T, g[j]);
    }
}

/// c_i      = mean_j(dy[i, j] * g[j] * x[i, j])
/// dx[i, j] = r_i * (dy[i, j] * g[j] - x[i, j] * r_i^2 * c_i) + alpha * dx_in[i, j]
/// dg[j]    = sum_i dy[i, j] * x[i, j] * r_i                  + alpha * dg_in[j]
/// The rows are walked in order, so the f64 sum of dg has one fixed order.
pub fn rmsnorm_ij_j_reverse(
    comptime T: type,
    x: []const T, g: []const T, dy: []const T,
    dx_in: ?[]const T, dg_in: ?[]const T,
    dx: []f64, dg: []f64,
    eps: f64, alpha: f64, m: usize, n: usize,
) void {
    const nf: f64 = @floatFromInt(n);
    @memset(dg, 0.0);
    for (0..m) |i| {
        const o = i * n;
        var ss: f64 = 0.0;
        var c: f64 = 0.0;
        for (0..n) |j| {
            const v = wide(T, x[o + j]);
            ss += v * v;
            c += wide(T, dy[o + j]) * wide(T, g[j]) * v;
        }
        const r = 1.0 / @sqrt(ss / nf + eps);
        c /= nf;
        for (0..n) |j| {
            const v = wide(T, x[o + j]);
            const t = wide(T, dy[o + j]);
            const old = if (dx_in) |p| alpha * wide(T, p[o + j]) else 0.0;
            dx[o + j] = r * (t * wide(T, g[j]) - v * r * r * c) + old;
            dg[j] += t * v * r;
        }
    }
    if (dg_in) |p| {
        for (dg, p) |*s, old| s.* += alpha * wide(T, old);
    }
}

// ---------------------------------------------------------------- what pins it where zig exists

test "softmax rows sum to one, -inf gives exact zero, one finite entry gives one" {
    const inf = std.math.inf(f32);
    const x = [_]f32{ 1.0, 2.0, 3.0, -inf, -inf, 0.5, -inf, -inf };
    var y: [8]f64 = undefined;
    softmax_ij_j(f32, &x, &y, 2, 4);
    try std.testing.expectApproxEqAbs(@as(f64, 1.0), y[0] + y[1] + y[2] + y[3], 1e-15);
    try std.testing.expectEqual(@as(f64, 0.0), y[3]);
    try std.testing.expectEqual(@as(f64, 1.0), y[5]);
}

test "rmsnorm with unit gain and no eps leaves rows of unit RMS" {
    const x = [_]f32{ 3.0, -4.0, 12.0, 5.0 };
    const g = [_]f32{ 1.0, 1.0 };
    var y: [4]f64 = undefined;
    rmsnorm_ij_j(f32, &x, &g, &y, 0.0, 2, 2);
    try std.testing.expectApproxEqAbs(@as(f64, 1.0), (y[0] * y[0] + y[1] * y[1]) / 2.0, 1e-15);
    try std.testing.expectApproxEqAbs(@as(f64, 1.0), (y[2] * y[2] + y[3] * y[3]) / 2.0, 1e-15);
}

test "selu is continuous at zero and linear above it" {
    try std.testing.expectEqual(@as(f64, 0.0), selu_value(0.0));
    try std.testing.expectApproxEqAbs(selu_scale * 2.0, selu_value(2.0), 1e-15);
    try std.testing.expectApproxEqAbs(-selu_scale * selu_alpha, selu_value(-800.0), 1e-15);
}
