//! Parameter structs for the device ops that the reference computes with host loops over `.raw` and that the
//! MI355X backend lifts to ops.  Append this file's declarations to src/device/opspec.zig: they follow that file's
//! pattern (`__name__`, `__type__`, slices for arrays) and use exactly the field names zig/hip_device.zig reads.
//! HostDevice gets the same names by moving its existing loops behind them (the line ranges are cited per struct),
//! so both devices stay interchangeable under DeviceReference.dispatch (src/device/device_reference.zig:15-27).
//!
//! `EdgePlan` in the *_planned structs is HipDevice.EdgePlan.

// ---- losses (src/nn/loss.zig) ----------------------------------------------------------------------------------

/// softmax + mean cross-entropy against one-hot (or soft) targets, probabilities kept for the backward pass:
/// src/nn/loss.zig:130-171 (`_softmax_fwd` + the loss loop).
pub fn smce_fwd(T: type) type {
    return struct {
        pub const __name__ = "smce_fwd";
        pub const __type__ = T;
        logits: []const T,
        target: []const T,
        probs: []T,
        loss: []T,
        rows: usize,
        cols: usize,
    };
}

/// grad += (probs - target) / rows: CceBwd.backward, src/nn/loss.zig:173-215.
pub fn smce_bwd(T: type) type {
    return struct {
        pub const __name__ = "smce_bwd";
        pub const __type__ = T;
        probs: []const T,
        target: []const T,
        grad: []T,
        rows: usize,
        cols: usize,
    };
}

/// smce_fwd and the backward of the scalar loss (upstream gradient 1) in one op.
pub fn smce_fwd_bwd(T: type) type {
    return struct {
        pub const __name__ = "smce_fwd_bwd";
        pub const __type__ = T;
        logits: []const T,
        target: []const T,
        probs: []T,
        loss: []T,
        grad: []T,
        rows: usize,
        cols: usize,
        accumulate: bool,
    };
}

/// The same loss from integer class labels: one pass over the logits, `lse` (per-row log-sum-exp) is what the
/// backward pass keeps instead of the probabilities.
pub fn smce_label_fwd(T: type) type {
    return struct {
        pub const __name__ = "smce_label_fwd";
        pub const __type__ = T;
        logits: []const T,
        labels: []const usize,
        lse: []T,
        loss: []T,
        rows: usize,
        cols: usize,
    };
}

pub fn smce_label_bwd(T: type) type {
    return struct {
        pub const __name__ = "smce_label_bwd";
        pub const __type__ = T;
        logits: []const T,
        labels: []const usize,
        lse: []const T,
        grad: []T,
        rows: usize,
        cols: usize,
        accumulate: bool,
    };
}

/// Row softmax and its backward: src/nn/loss.zig:217-257.
pub fn softmax_fwd(T: type) type {
    return struct {
        pub const __name__ = "softmax_fwd";
        pub const __type__ = T;
        x: []const T,
        y: []T,
        rows: usize,
        cols: usize,
    };
}

pub fn softmax_bwd(T: type) type {
    return struct {
        pub const __name__ = "softmax_bwd";
        pub const __type__ = T;
        y: []const T,
        y_g: []const T,
        x_g: []T,
        rows: usize,
        cols: usize,
    };
}

/// mean smooth-L1: src/nn/loss.zig:259-305.
pub fn smooth_l1_fwd(T: type) type {
    return struct {
        pub const __name__ = "smooth_l1_fwd";
        pub const __type__ = T;
        pred: []const T,
        target: []const T,
        beta: T,
        loss: []T,
    };
}

pub fn smooth_l1_bwd(T: type) type {
    return struct {
        pub const __name__ = "smooth_l1_bwd";
        pub const __type__ = T;
        pred: []const T,
        target: []const T,
        grad: []T,
        beta: T,
    };
}

pub fn smooth_l1_fwd_bwd(T: type) type {
    return struct {
        pub const __name__ = "smooth_l1_fwd_bwd";
        pub const __type__ = T;
        pred: []const T,
        target: []const T,
        grad: []T,
        beta: T,
        loss: []T,
        accumulate: bool,
    };
}

/// mean squared error: src/nn/loss.zig:94-127.
pub fn mse_fwd(T: type) type {
    return struct {
        pub const __name__ = "mse_fwd";
        pub const __type__ = T;
        pred: []const T,
        target: []const T,
        loss: []T,
    };
}

pub fn mse_bwd(T: type) type {
    return struct {
        pub const __name__ = "mse_bwd";
        pub const __type__ = T;
        pred: []const T,
        target: []const T,
        grad: []T,
    };
}

// ---- optimizers (src/nn/optim.zig) -----------------------------------------------------------------------------

/// Per-tensor clip + `param -= lr * grad`: SGD.update, src/nn/optim.zig:100-122.
pub fn sgd_step(T: type) type {
    return struct {
        pub const __name__ = "sgd_step";
        pub const __type__ = T;
        param: []T,
        grad: []T,
        lr: T,
        clip: bool,
        max_norm: T,
        delta: T,
    };
}

/// Per-tensor clip + Adam update with the per-tensor counter `t`: Adam.update, src/nn/optim.zig:177-234.
pub fn adam_step(T: type) type {
    return struct {
        pub const __name__ = "adam_step";
        pub const __type__ = T;
        param: []T,
        grad: []T,
        m: []T,
        v: []T,
        t: usize,
        lr: T,
        beta1: T,
        beta2: T,
        epsilon: T,
        clip: bool,
        max_norm: T,
        delta: T,
    };
}

/// Adam update whose step size `lr_t` is read from memory when the kernel runs (one element, device or pinned host).
pub fn adam_step_at(T: type) type {
    return struct {
        pub const __name__ = "adam_step_at";
        pub const __type__ = T;
        param: []T,
        grad: []T,
        m: []T,
        v: []T,
        lr_t: []const T,
        beta1: T,
        beta2: T,
        epsilon: T,
        clip: bool,
        max_norm: T,
        delta: T,
    };
}

/// Optimizer.step() over the whole parameter list, optionally followed by zero_grad().
pub fn sgd_step_multi(T: type) type {
    return struct {
        pub const __name__ = "sgd_step_multi";
        pub const __type__ = T;
        params: []const [*]T,
        grads: []const [*]T,
        lens: []const usize,
        lr: T,
        clip: bool,
        max_norm: T,
        delta: T,
        zero_grads: bool,
    };
}

pub fn adam_step_multi(T: type) type {
    return struct {
        pub const __name__ = "adam_step_multi";
        pub const __type__ = T;
        params: []const [*]T,
        grads: []const [*]T,
        ms: []const [*]T,
        vs: []const [*]T,
        lens: []const usize,
        lr_t: []const T,
        lr_t_in_memory: bool,
        beta1: T,
        beta2: T,
        epsilon: T,
        clip: bool,
        max_norm: T,
        delta: T,
        zero_grads: bool,
    };
}

// ---- indexing ----------------------------------------------------------------------------------------------------

/// First index of the maximum along `dim` (the examples' accuracy loops: std.mem.indexOfMax on a host row,
/// examples/mnist/src/main-simple.zig:124-125).
pub fn argmax_along(T: type) type {
    return struct {
        pub const __name__ = "argmax_along";
        pub const __type__ = T;
        x: []const T,
        x_shape: []const usize,
        y: []usize,
        dim: usize,
    };
}

/// The offsets loop of NDArray.gather, src/ndarray.zig:607-624.
pub fn gather_offsets(T: type) type {
    return struct {
        pub const __name__ = "gather_offsets";
        pub const __type__ = T;
        src_shape: []const usize,
        idx_shape: []const usize,
        indices: []const usize,
        dim: usize,
        offsets: []usize,
        check: bool,
    };
}

/// NDArray.gather as one op: offsets and gathered values, src/ndarray.zig:593-633.
pub fn gather(T: type) type {
    return struct {
        pub const __name__ = "gather";
        pub const __type__ = T;
        src: []const T,
        src_shape: []const usize,
        idx_shape: []const usize,
        indices: []const usize,
        dim: usize,
        offsets: []usize,
        dst: []T,
        check: bool,
    };
}

/// NDTensor.index_select and its backward, src/ndtensor.zig:1437-1513 (one mem_copy / add per index there).
pub fn index_select_fwd(T: type) type {
    return struct {
        pub const __name__ = "index_select_fwd";
        pub const __type__ = T;
        src: []const T,
        indices: []const usize,
        stride: usize,
        dst: []T,
    };
}

pub fn index_select_bwd(T: type) type {
    return struct {
        pub const __name__ = "index_select_bwd";
        pub const __type__ = T;
        y_grad: []const T,
        indices: []const usize,
        stride: usize,
        x_grad: []T,
    };
}

// ---- the scatter ops on an edge plan built once -------------------------------------------------------------------

pub fn scatter_add_planned(T: type) type {
    return struct {
        pub const __name__ = "scatter_add_planned";
        pub const __type__ = T;
        src: []const T,
        plan: *const EdgePlan,
        dst: []T,
        accumulate: bool,
    };
}

pub fn scatter_gcn_deg_scaled_planned(T: type) type {
    return struct {
        pub const __name__ = "scatter_gcn_deg_scaled_planned";
        pub const __type__ = T;
        dst: []T,
        h: []const T,
        deg: []const T,
        plan: *const EdgePlan,
        bias: ?[]const T,
        relu: bool,
        stride: usize,
        accumulate: bool,
    };
}

pub fn scatter_gcn_deg_scaled_bwd_planned(T: type) type {
    return struct {
        pub const __name__ = "scatter_gcn_deg_scaled_bwd_planned";
        pub const __type__ = T;
        grad_output: []const T,
        h: []const T,
        deg: []const T,
        plan: *const EdgePlan,
        grad_h: []T,
        grad_deg: ?[]T,
        stride: usize,
        accumulate: bool,
    };
}

// ---- a Linear layer in one op (examples/mnist/src/model.zig:104-110, src/ndtensor.zig:1092-1136) ----------------------

pub fn linear_fwd(T: type) type {
    return struct {
        pub const __name__ = "linear_fwd";
        pub const __type__ = T;
        x: []const T,
        w: []const T,
        bias: ?[]const T,
        y: []T,
        batch: usize,
        fan_in: usize,
        fan_out: usize,
        relu: bool,
    };
}

pub fn linear_bwd_input(T: type) type {
    return struct {
        pub const __name__ = "linear_bwd_input";
        pub const __type__ = T;
        gy: []const T,
        w: []const T,
        act_in: ?[]const T,
        gx: []T,
        batch: usize,
        fan_in: usize,
        fan_out: usize,
        accumulate: bool,
    };
}

pub fn linear_bwd(T: type) type {
    return struct {
        pub const __name__ = "linear_bwd";
        pub const __type__ = T;
        gy: []const T,
        x: []const T,
        w: []const T,
        act_in: ?[]const T,
        gw: []T,
        gb: ?[]T,
        gx: ?[]T,
        batch: usize,
        fan_in: usize,
        fan_out: usize,
    };
}

const EdgePlan = @import("hip_device.zig").EdgePlan;
