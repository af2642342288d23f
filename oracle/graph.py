"""CPU restatement of the reference's sequential operator chain and SGD update block.

TEST INFRASTRUCTURE ONLY (see oracle.c).  numpy arrays + the C oracle; one class per reference
operator, same method names and the same order of operations as the Rust sources:

  Conv2dOperator::forward/backward ........ src/operator/mod.rs:1663-1795
  AffineOperator::forward/backward ........ src/operator/mod.rs:1075-1176
  Pool2dOperator::forward/backward ........ src/operator/mod.rs:2103-2123
  SoftmaxKLLossOperator ................... src/operator/loss.rs:118-261
  regularize / accumulate_grads / update_params / update_params2 / reset
                                            src/operator/mod.rs:1178-1236, 1355-1363
  SequentialOperatorWorker fan-out ........ src/operator/worker.rs:356-477
  SgdOpt update block ..................... src/opt/sgd/new.rs:345-495, 623-633
  SgdOpt::train / validate loops .......... src/opt/sgd/new.rs:209-344, 495-766
  second-generation layer methods backward(batch, scale), descend, reset_gradients
                                            src/layer_new.rs:537-617, 1044-1154
  PipelineArchWorker fan-out .............. src/arch_new.rs:527-552
  SgdOptimization minibatch block ......... src/opt_new.rs:279-325
  BNormConv2d / StackResConv2d / ProjStackResConv2d operators
                                            src/operator/conv.rs:461-912, 1497-2182, 2935-3560

`fast=True` switches the contractions to the fp32 im2col + SGEMM family (the timed CPU baseline);
the default is the fp64-accumulating family (the parity checker).
"""
import numpy as np

import oracle as O


class _Params:
    def __init__(self, w_shape, b_len):
        self.weights = np.zeros(w_shape, np.float32)
        self.bias = np.zeros((b_len,), np.float32)
        self.grad_weights = np.zeros(w_shape, np.float32)
        self.grad_bias = np.zeros((b_len,), np.float32)
        self.acc_grad_weights = np.zeros(w_shape, np.float32)
        self.acc_grad_bias = np.zeros((b_len,), np.float32)
        self.save_weights = np.zeros(w_shape, np.float32)
        self.save_bias = np.zeros((b_len,), np.float32)

    def regularize(self, l2):
        assert l2 >= 0.0
        if l2 > 0.0:  # weights *and bias*: mod.rs:1186-1189
            O.saxpy(l2, self.weights, self.grad_weights)
            O.saxpy(l2, self.bias, self.grad_bias)

    def accumulate_grads(self, scale, momentum):
        O.sscal(momentum, self.acc_grad_weights)
        O.sscal(momentum, self.acc_grad_bias)
        O.saxpy(scale, self.grad_weights, self.acc_grad_weights)
        O.saxpy(scale, self.grad_bias, self.acc_grad_bias)

    def update_params(self, scale):
        O.saxpy(scale, self.acc_grad_weights, self.weights)
        O.saxpy(scale, self.acc_grad_bias, self.bias)

    def update_params2(self, grad_scale, update_scale):
        if grad_scale != 0.0:
            O.saxpy(grad_scale, self.grad_weights, self.weights)
            O.saxpy(grad_scale, self.grad_bias, self.bias)
        if update_scale != 0.0:
            O.saxpy(update_scale, self.acc_grad_weights, self.weights)
            O.saxpy(update_scale, self.acc_grad_bias, self.bias)

    def save_params(self):
        self.save_weights[...] = self.weights
        self.save_bias[...] = self.bias

    def restore_params(self):
        self.weights[...] = self.save_weights
        self.bias[...] = self.save_bias

    def reset(self):
        O.sscal(0.0, self.grad_weights)
        O.sscal(0.0, self.grad_bias)

    # second generation: the gradient buffers double as the momentum buffers
    def descend(self, scale, l2):
        """g += l2*W (weights and bias); W -= scale*g: layer_new.rs:596-617 (affine), 1133-1154 (conv)."""
        assert l2 >= 0.0
        if l2 > 0.0:
            O.saxpy(l2, self.weights, self.grad_weights)
            O.saxpy(l2, self.bias, self.grad_bias)
        O.saxpy(-scale, self.grad_weights, self.weights)
        O.saxpy(-scale, self.grad_bias, self.bias)

    def reset_gradients(self, scale):
        """g *= scale: layer_new.rs:589-594, 1126-1131."""
        O.sscal(scale, self.grad_weights)
        O.sscal(scale, self.grad_bias)


class Conv2dOperator:
    kind = "Conv2dOperator"

    def __init__(self, batch, in_dims, conv_size, conv_stride, conv_pad, out_channels, act_func, fast=False):
        w, h, c = in_dims
        self.x_shape = (batch, c, h, w)
        self.stride, self.pad, self.act, self.fast = conv_stride, conv_pad, act_func, fast
        self.bf16_forward = False   # forward multiplies operands rounded to bf16 (the build's inference math mode)
        self.p = _Params((out_channels, c, conv_size, conv_size), out_channels)
        P = O.out_dim(h, conv_size, conv_stride, conv_pad)
        Q = O.out_dim(w, conv_size, conv_stride, conv_pad)
        self.out_dims = (Q, P, out_channels)
        self.out_act = np.zeros((batch, out_channels, P, Q), np.float32)
        self.out_delta = np.zeros_like(self.out_act)

    def forward(self, in_act):
        self.in_act = in_act = np.ascontiguousarray(in_act.reshape(self.x_shape))   # buffers are flat: any operator may precede
        if self.bf16_forward:
            O.conv2d_fwd(O.round_bf16(in_act), O.round_bf16(self.p.weights), self.stride, self.pad, y=self.out_act)
        elif self.fast:
            self.out_act = O.fast_conv2d_fwd(in_act, self.p.weights, self.stride, self.pad)
        else:
            O.conv2d_fwd(in_act, self.p.weights, self.stride, self.pad, y=self.out_act)
        O.add_bias_nchw(self.p.bias, self.out_act)
        if self.act == "Rect":
            O.rect_inplace(self.out_act)
        return self.out_act

    def backward(self, want_in_delta, scale=1.0):
        """`scale`: the alpha of backward_filter / backward_bias; 1 in the operator generation (mod.rs:1765-1781), the
        caller's `scale` in Conv2dLayer::backward (layer_new.rs:1093-1108)."""
        if self.act == "Rect":
            O.rect_backprop_inplace(self.out_act, self.out_delta)
        if self.fast:
            assert scale == 1.0
            O.fast_conv2d_bwd_filter(self.in_act, self.out_delta, self.p.grad_weights, self.stride, self.pad)
        else:
            O.conv2d_bwd_filter(self.in_act, self.out_delta, self.p.weights.shape, self.stride, self.pad, scale, 1.0,
                                self.p.grad_weights)
        O.conv2d_bwd_bias(self.out_delta, scale, 1.0, self.p.grad_bias)
        if not want_in_delta:
            return None
        if self.fast:
            return O.fast_conv2d_bwd_data(self.p.weights, self.out_delta, self.x_shape, self.stride, self.pad)
        return O.conv2d_bwd_data(self.p.weights, self.out_delta, self.x_shape, self.stride, self.pad)


class AffineOperator:
    kind = "AffineOperator"

    def __init__(self, batch, in_channels, out_channels, act_func, fast=False):
        self.batch, self.i, self.o, self.act, self.fast = batch, in_channels, out_channels, act_func, fast
        self.p = _Params((out_channels, in_channels), out_channels)  # (in, out) column-major = [out][in]
        self.out_dims = (1, 1, out_channels)
        self.out_act = np.zeros((batch, out_channels), np.float32)
        self.out_delta = np.zeros_like(self.out_act)

    def forward(self, in_act):
        x = np.ascontiguousarray(in_act.reshape(self.batch, self.i))
        self.in_act = x
        if self.fast:
            self.out_act = O.fast_gemm_rm(x, self.p.weights, transB=True)
        else:  # out_act(out,B) = W(in,out)^T * X(in,B)
            O.sgemm(1, 0, self.o, self.batch, self.i, 1.0, self.p.weights, self.i, x, self.i, 0.0, self.out_act, self.o)
        O.add_bias_nchw(self.p.bias, self.out_act)
        if self.act == "Rect":
            O.rect_inplace(self.out_act)
        return self.out_act

    def backward(self, want_in_delta, scale=1.0):
        """AffineLayer::backward takes `scale` and accumulates both gradients with factor 1.0 (layer_new.rs:583-584)."""
        if self.act == "Rect":
            O.rect_backprop_inplace(self.out_act, self.out_delta)
        if self.fast:
            O.fast_gemm_rm(self.out_delta, self.in_act, transA=True, out=self.p.grad_weights, accumulate=True)
        else:  # dW(in,out) += X(in,B) * dY(out,B)^T
            O.sgemm(0, 1, self.i, self.o, self.batch, 1.0, self.in_act, self.i, self.out_delta, self.o, 1.0,
                    self.p.grad_weights, self.i)
        O.conv2d_bwd_bias(self.out_delta, 1.0, 1.0, self.p.grad_bias)  # 1(1,B) * dY^T
        if not want_in_delta:
            return None
        if self.fast:
            return O.fast_gemm_rm(self.out_delta, self.p.weights)
        dx = np.zeros((self.batch, self.i), np.float32)  # dX(in,B) = W(in,out) * dY(out,B)
        O.sgemm(0, 0, self.i, self.batch, self.o, 1.0, self.p.weights, self.i, self.out_delta, self.o, 0.0, dx, self.i)
        return dx


class Pool2dOperator:
    kind = "Pool2dOperator"
    p = None

    def __init__(self, batch, in_dims, pool_size, pool_stride, pool_pad, pool_op, ceil_mode=False):
        w, h, c = in_dims
        self.x_shape = (batch, c, h, w)
        self.k, self.st, self.pad = pool_size, pool_stride, pool_pad
        self.mode = O.POOL_MAX if pool_op == "Max" else O.POOL_AVG
        self.rounding = O.ROUND_CEIL if ceil_mode else O.ROUND_FLOOR
        g = O.pool_geom(self.x_shape, pool_size, pool_stride, pool_pad, self.mode, self.rounding)
        shp = O.pool_out_shape(g)
        self.out_dims = (shp[3], shp[2], c)
        self.out_act = np.zeros(shp, np.float32)
        self.out_delta = np.zeros(shp, np.float32)

    def forward(self, in_act):
        self.in_act = np.ascontiguousarray(in_act.reshape(self.x_shape))
        self.out_act = O.pool2d_fwd(self.in_act, self.k, self.st, self.pad, self.mode, self.rounding)
        return self.out_act

    def backward(self, want_in_delta):
        if not want_in_delta:
            return None
        return O.pool2d_bwd(self.in_act, self.out_act, self.out_delta, self.k, self.st, self.pad, self.mode, self.rounding)


class DropoutOperator:
    """src/operator/mod.rs:2134-2255.  `rnd` (the uniform samples of this forward) is set by the caller: the
    reference draws them from a device generator whose stream cannot be reproduced."""
    kind = "DropoutOperator"
    p = None

    def __init__(self, batch, channels, drop_ratio):
        self.x_shape = (batch, channels)
        self.ratio = drop_ratio
        self.rnd = None
        self.training = True
        self.out_act = np.zeros(self.x_shape, np.float32)
        self.out_delta = np.zeros(self.x_shape, np.float32)

    def forward(self, in_act):
        self.in_act = np.ascontiguousarray(in_act.reshape(self.x_shape))
        if not self.training:
            self.out_act = self.in_act.copy()
            return self.out_act
        self.out_act, self.mask = O.dropout(self.in_act, self.ratio, 1.0, self.rnd.reshape(self.x_shape))
        return self.out_act

    def backward(self, want_in_delta):
        if not want_in_delta:
            return None
        return O.dropout_backprop(self.out_delta.reshape(self.x_shape), 1.0, self.mask)


class LocalResNormOperator:
    """Cross-channel local response normalisation (`local_res_norm` of the .model grammar)."""
    kind = "LocalResNormOperator"
    p = None

    def __init__(self, batch, in_dims, cross_size, scale, power, min_div):
        w, h, c = in_dims
        self.x_shape = (batch, c, h, w)
        self.args = (cross_size, scale, power, min_div)
        self.out_act = np.zeros(self.x_shape, np.float32)
        self.out_delta = np.zeros(self.x_shape, np.float32)

    def forward(self, in_act):
        self.in_act = np.ascontiguousarray(in_act.reshape(self.x_shape))
        self.out_act, _ = O.lrn_fwd(self.in_act, *self.args)
        return self.out_act

    def backward(self, want_in_delta):
        if not want_in_delta:
            return None
        return O.lrn_bwd(self.in_act, self.out_delta.reshape(self.x_shape), *self.args)


class _BNormUnit:
    """conv (no bias) + spatial batch norm with the reference's buffers and update rules per unit
    (src/operator/conv.rs:133-160 buffers; :640-911 regularize the filter only, accumulate / update / save / restore /
    reset the filter, scale and bias; the moving statistics travel with save / restore)."""

    def __init__(self, batch, in_dims, size, stride, pad, out_channels, fast=False):
        w, h, c = in_dims
        self.x_shape = (batch, c, h, w)
        self.stride, self.pad, self.fast = stride, pad, fast
        f = np.float32
        self.weights = np.zeros((out_channels, c, size, size), f)
        self.grad_weights, self.acc_grad_weights, self.save_weights = (np.zeros_like(self.weights) for _ in range(3))
        K = out_channels
        self.scale, self.bias = np.ones(K, f), np.zeros(K, f)
        self.running_mean, self.running_ivar = np.zeros(K, f), np.ones(K, f)
        self.scale_grad, self.bias_grad, self.acc_scale_grad, self.acc_bias_grad = (np.zeros(K, f) for _ in range(4))
        self.save_scale, self.save_bias, self.save_running_mean, self.save_running_ivar = (np.zeros(K, f) for _ in range(4))
        self.cached_mean, self.cached_ivar = np.zeros(K, f), np.zeros(K, f)
        P, Q = O.out_dim(h, size, stride, pad), O.out_dim(w, size, stride, pad)
        self.out_dims = (Q, P, K)
        self.pre_act = np.zeros((batch, K, P, Q), f)
        self.bf16_forward = False

    def forward(self, in_act, out, beta_out, training, t, mov_avg, epsilon):
        """Returns beta_out*out + BN(conv(in_act)) (forward_training / forward_inference, conv.rs:493-535)."""
        in_act = np.ascontiguousarray(in_act.reshape(self.x_shape))
        self.in_act = in_act
        if self.bf16_forward:
            O.conv2d_fwd(O.round_bf16(in_act), O.round_bf16(self.weights), self.stride, self.pad, y=self.pre_act)
        elif self.fast:
            self.pre_act = O.fast_conv2d_fwd(in_act, self.weights, self.stride, self.pad)
        else:
            O.conv2d_fwd(in_act, self.weights, self.stride, self.pad, y=self.pre_act)
        if training:
            ema = O.bnorm_mov_avg_at_iter(mov_avg[0], mov_avg[1], t)
            y, self.cached_mean, self.cached_ivar, self.running_mean, self.running_ivar = O.bnorm_fwd_train(
                self.pre_act, self.scale, self.bias, self.running_mean, self.running_ivar, ema, epsilon, 1.0, beta_out, out)
            return y
        return O.bnorm_fwd_infer(self.pre_act, self.scale, self.bias, self.running_mean, self.running_ivar, 1.0, beta_out, out)

    def backward_params(self, out_delta):
        """pre_delta = dBN(out_delta), scale / bias gradients accumulated (beta 1); grad_weights += dconv (conv.rs:594-618)."""
        self.pre_delta, ds, db = O.bnorm_bwd(self.pre_act, out_delta, self.scale, self.cached_mean, self.cached_ivar)
        self.scale_grad = (self.scale_grad + ds).astype(np.float32)
        self.bias_grad = (self.bias_grad + db).astype(np.float32)
        if self.fast:
            O.fast_conv2d_bwd_filter(self.in_act, self.pre_delta, self.grad_weights, self.stride, self.pad)
        else:
            O.conv2d_bwd_filter(self.in_act, self.pre_delta, self.weights.shape, self.stride, self.pad, 1.0, 1.0,
                                self.grad_weights)

    def backward_data(self, beta=0.0, dx=None):
        if self.fast:
            d = O.fast_conv2d_bwd_data(self.weights, self.pre_delta, self.x_shape, self.stride, self.pad)
            return d if beta == 0.0 else (d + np.float32(beta) * dx).astype(np.float32)
        return O.conv2d_bwd_data(self.weights, self.pre_delta, self.x_shape, self.stride, self.pad, 1.0, beta, dx)

    def _triples(self):
        return ((self.weights, self.grad_weights, self.acc_grad_weights), (self.scale, self.scale_grad, self.acc_scale_grad),
                (self.bias, self.bias_grad, self.acc_bias_grad))

    def regularize(self, l2):
        assert l2 >= 0.0
        if l2 > 0.0:
            O.saxpy(l2, self.weights, self.grad_weights)

    def accumulate_grads(self, scale, momentum):
        for _, g, v in self._triples():
            O.sscal(momentum, v)
            O.saxpy(scale, g, v)

    def update_params(self, scale):
        for w, _, v in self._triples():
            O.saxpy(scale, v, w)

    def update_params2(self, grad_scale, update_scale):
        if grad_scale != 0.0:
            for w, g, _ in self._triples():
                O.saxpy(grad_scale, g, w)
        if update_scale != 0.0:
            for w, _, v in self._triples():
                O.saxpy(update_scale, v, w)

    def save_params(self):
        self.save_weights[...] = self.weights
        self.save_scale[...], self.save_bias[...] = self.scale, self.bias
        self.save_running_mean[...], self.save_running_ivar[...] = self.running_mean, self.running_ivar

    def restore_params(self):
        self.weights[...] = self.save_weights
        self.scale[...], self.bias[...] = self.save_scale, self.save_bias
        self.running_mean, self.running_ivar = self.save_running_mean.copy(), self.save_running_ivar.copy()

    def reset(self):
        for _, g, _ in self._triples():
            O.sscal(0.0, g)

    def params_len(self):
        return self.weights.size + 4 * self.scale.size


class _UnitsParams:
    """What SequentialOperatorWorker fans the SGD methods out to, for an operator made of several units."""

    def __init__(self, units):
        self.units = units

    def params_len(self):
        return sum(u.params_len() for u in self.units)

    def __getattr__(self, name):
        if name in ("regularize", "accumulate_grads", "update_params", "update_params2", "save_params", "restore_params", "reset"):
            return lambda *a: [getattr(u, name)(*a) for u in self.units]
        raise AttributeError(name)


class BNormConv2dOperator:
    """out = act(BN(conv(in))) (src/operator/conv.rs:461-640)."""
    kind = "BNormConv2dOperator"
    wants_phase = True

    def __init__(self, batch, in_dims, conv_size, conv_stride, conv_pad, out_channels, act_func, mov_avg=("Exponential", 0.1),
                 epsilon=1e-5, fast=False):
        self.units = [_BNormUnit(batch, in_dims, conv_size, conv_stride, conv_pad, out_channels, fast)]
        self.p = _UnitsParams(self.units)
        self.act, self.mov_avg, self.epsilon = act_func, mov_avg, epsilon
        self.out_dims = self.units[0].out_dims
        self.out_act = np.zeros_like(self.units[0].pre_act)
        self.out_delta = np.zeros_like(self.out_act)

    def forward(self, in_act, training=True, t=0):
        self.out_act = self.units[0].forward(in_act, None, 0.0, training, t, self.mov_avg, self.epsilon)
        if self.act == "Rect":
            O.rect_inplace(self.out_act)
        return self.out_act

    def backward(self, want_in_delta):
        if self.act == "Rect":
            O.rect_backprop_inplace(self.out_act, self.out_delta)
        self.units[0].backward_params(self.out_delta)
        return self.units[0].backward_data() if want_in_delta else None


class StackResConv2dOperator:
    """out = act(in + BN2(conv2(act(BN1(conv1(in)))))), 3x3 / stride 1 / pad 1 (src/operator/conv.rs:1497-1830)."""
    kind = "StackResConv2dOperator"
    wants_phase = True

    def __init__(self, batch, in_dims, act_func, mov_avg=("Exponential", 0.1), epsilon=1e-5, fast=False):
        c = in_dims[2]
        self.units = [_BNormUnit(batch, in_dims, 3, 1, 1, c, fast), _BNormUnit(batch, in_dims, 3, 1, 1, c, fast)]
        self.p = _UnitsParams(self.units)
        self.act, self.mov_avg, self.epsilon = act_func, mov_avg, epsilon
        self.out_dims = in_dims
        self.out_act = np.zeros_like(self.units[0].pre_act)
        self.out_delta = np.zeros_like(self.out_act)

    def forward(self, in_act, training=True, t=0):
        u1, u2 = self.units
        self.mid_act = u1.forward(in_act, None, 0.0, training, t, self.mov_avg, self.epsilon)
        if self.act == "Rect":
            O.rect_inplace(self.mid_act)
        self.out_act = u2.forward(self.mid_act, in_act.reshape(self.out_act.shape), 1.0, training, t, self.mov_avg, self.epsilon)
        if self.act == "Rect":
            O.rect_inplace(self.out_act)
        return self.out_act

    def backward(self, want_in_delta):
        u1, u2 = self.units
        if self.act == "Rect":
            O.rect_backprop_inplace(self.out_act, self.out_delta)
        u2.backward_params(self.out_delta)
        self.mid_delta = u2.backward_data()
        if self.act == "Rect":
            O.rect_backprop_inplace(self.mid_act, self.mid_delta)
        u1.backward_params(self.mid_delta)
        if not want_in_delta:
            return None
        return u1.backward_data(1.0, self.out_delta.reshape(u1.x_shape).copy())


class ProjStackResConv2dOperator:
    """out = act(BN2(conv2(act(BN1(conv1(in))))) + BN3(conv3(in))): conv1 3x3 / stride s / pad 1, conv2 3x3 / 1 / 1,
    conv3 1x1 / stride s / pad 0, s = 1 or 2 from the two extents (src/operator/conv.rs:2331-2338, 2935-3385)."""
    kind = "ProjStackResConv2dOperator"
    wants_phase = True

    def __init__(self, batch, in_dims, out_dims, act_func, mov_avg=("Exponential", 0.1), epsilon=1e-5, fast=False):
        if in_dims[:2] == out_dims[:2]:
            s = 1
        else:
            assert in_dims[0] == 2 * out_dims[0] and in_dims[1] == 2 * out_dims[1]
            s = 2
        oc = out_dims[2]
        self.units = [_BNormUnit(batch, in_dims, 3, s, 1, oc, fast), _BNormUnit(batch, out_dims, 3, 1, 1, oc, fast),
                      _BNormUnit(batch, in_dims, 1, s, 0, oc, fast)]
        self.p = _UnitsParams(self.units)
        self.act, self.mov_avg, self.epsilon = act_func, mov_avg, epsilon
        self.out_dims = out_dims
        self.out_act = np.zeros_like(self.units[1].pre_act)
        self.out_delta = np.zeros_like(self.out_act)

    def forward(self, in_act, training=True, t=0):
        u1, u2, u3 = self.units
        self.mid_act = u1.forward(in_act, None, 0.0, training, t, self.mov_avg, self.epsilon)
        if self.act == "Rect":
            O.rect_inplace(self.mid_act)
        out = u2.forward(self.mid_act, None, 0.0, training, t, self.mov_avg, self.epsilon)
        self.out_act = u3.forward(in_act, out, 1.0, training, t, self.mov_avg, self.epsilon)
        if self.act == "Rect":
            O.rect_inplace(self.out_act)
        return self.out_act

    def backward(self, want_in_delta):
        u1, u2, u3 = self.units
        if self.act == "Rect":
            O.rect_backprop_inplace(self.out_act, self.out_delta)
        u2.backward_params(self.out_delta)
        self.mid_delta = u2.backward_data()
        if self.act == "Rect":
            O.rect_backprop_inplace(self.mid_act, self.mid_delta)
        u1.backward_params(self.mid_delta)
        u3.backward_params(self.out_delta)
        if not want_in_delta:
            return None
        return u3.backward_data(1.0, u1.backward_data())


class SequentialOperatorWorker:
    """layers: list of tuples mirroring the SequentialOperatorConfig builder calls, e.g.
    ("conv2d", in_dims, size, stride, pad, out_channels, act), ("pool2d", in_dims, size, stride, pad, op, ceil),
    ("affine", in, out, act); num_categories closes the chain with SoftmaxKLLoss."""

    def __init__(self, layers, num_categories, batch, fast=False, bnorm_mov_avg=("Exponential", 0.1), bnorm_epsilon=1e-5):
        self.batch, self.C = batch, num_categories
        self.hidden = []
        if isinstance(bnorm_mov_avg, str):
            bnorm_mov_avg = (bnorm_mov_avg, 0.0)
        bnorm = {"mov_avg": bnorm_mov_avg, "epsilon": bnorm_epsilon, "fast": fast}
        for l in layers:
            if l[0] == "conv2d":
                self.hidden.append(Conv2dOperator(batch, *l[1:], fast=fast))
            elif l[0] == "affine":
                self.hidden.append(AffineOperator(batch, *l[1:], fast=fast))
            elif l[0] == "pool2d":
                self.hidden.append(Pool2dOperator(batch, *l[1:]))
            elif l[0] == "dropout":
                self.hidden.append(DropoutOperator(batch, *l[1:]))
            elif l[0] == "local_res_norm":
                self.hidden.append(LocalResNormOperator(batch, *l[1:]))
            elif l[0] == "bnorm_conv2d":
                self.hidden.append(BNormConv2dOperator(batch, *l[1:], **bnorm))
            elif l[0] == "stack_res_conv2d":
                self.hidden.append(StackResConv2dOperator(batch, *l[1:], **bnorm))
            elif l[0] == "proj_stack_res_conv2d":
                self.hidden.append(ProjStackResConv2dOperator(batch, *l[1:], **bnorm))
            else:
                raise ValueError(l[0])
        self.labels = np.zeros((batch,), np.int32)
        self.weights = np.zeros((batch,), np.float32)
        self.out_cats = np.zeros((batch,), np.int32)

    def params_len(self):
        return sum(op.p.params_len() if hasattr(op.p, "params_len") else op.p.weights.size + op.p.bias.size
                   for op in self.hidden if op.p is not None)

    def stage_batch(self, labels, weight):
        self.labels[...] = labels
        self.weights[...] = weight

    def forward(self, frames, training=True, t=0):
        """`training`, `t`: the OpPhase the batch-normalised operators read (Training{t} or Inference)."""
        act = frames
        for op in self.hidden:
            act = op.forward(act, training, t) if getattr(op, "wants_phase", False) else op.forward(act)
        self.out_values = O.softmax_fwd(np.ascontiguousarray(act.reshape(self.batch, self.C)))

    def store_output_categories(self):
        _, self.out_cats = O.blockreduce_argmax(self.out_values)
        return self.out_cats

    def store_loss(self):
        loss1 = O.softmax_kl_loss1(self.out_values, self.labels, self.weights)
        return float(O.blockreduce_sum(loss1.reshape(1, -1))[0])

    def accuracy_count(self):
        return O.accuracy_count(self.labels, self.out_cats)

    def backward(self):
        delta = O.softmax_kl_backward(self.out_values, self.labels, self.weights)
        for i in range(len(self.hidden) - 1, -1, -1):
            op = self.hidden[i]
            op.out_delta = np.ascontiguousarray(delta.reshape(op.out_act.shape))
            delta = op.backward(want_in_delta=i > 0)  # the input operator exposes no deltas (mod.rs:632-634)

    def backward_scaled(self, scale):
        """PipelineArchWorker::backward(batch, scale), arch_new.rs:534-539: the loss layer ignores the scale
        (layer_new.rs:1933); operators with parameters receive it, the others have nothing to scale."""
        delta = O.softmax_kl_backward(self.out_values, self.labels, self.weights)
        for i in range(len(self.hidden) - 1, -1, -1):
            op = self.hidden[i]
            op.out_delta = np.ascontiguousarray(delta.reshape(op.out_act.shape))
            if op.kind in ("Conv2dOperator", "AffineOperator"):
                delta = op.backward(want_in_delta=i > 0, scale=scale)
            else:
                delta = op.backward(want_in_delta=i > 0)

    def descend(self, scale, l2): self._each("descend", scale, l2)              # arch_new.rs:541-545
    def reset_gradients(self, momentum): self._each("reset_gradients", momentum)  # arch_new.rs:547-551

    # second-generation loss bookkeeping, layer_new.rs:2103-2134: out_loss sums the batches until reset_loss
    def reset_loss(self):
        self.acc_loss = np.zeros((1,), np.float32)

    def accumulate_loss(self):
        loss1 = O.softmax_kl_loss1(self.out_values, self.labels, self.weights)
        O.blockreduce_sum(loss1.reshape(1, -1), 1.0, self.acc_loss)

    def _each(self, fn, *a):
        for op in self.hidden:
            if op.p is not None:
                getattr(op.p, fn)(*a)

    def regularize(self, l2): self._each("regularize", l2)
    def accumulate_grads(self, scale, momentum): self._each("accumulate_grads", scale, momentum)
    def update_params(self, scale): self._each("update_params", scale)
    def update_params2(self, g, u): self._each("update_params2", g, u)
    def save_params(self): self._each("save_params")
    def restore_params(self): self._each("restore_params")
    def reset(self): self._each("reset")


def step_size_at(schedule, t):
    """StepSizeSchedule::at_iter, src/opt/sgd/mod.rs:82-132."""
    kind = schedule["kind"]
    s, it = schedule.get("steps", []), schedule.get("iters", [])
    if kind == "Constant":
        return s[0]
    if kind == "Anneal1":
        return s[0] if t < it[1] else s[1]
    if kind == "Anneal2":
        return s[0] if t < it[1] else s[1] if t < it[2] else s[2]
    if kind == "Anneal4":
        return s[0] if t < it[1] else s[1] if t < it[2] else s[2] if t < it[3] else s[3] if t < it[4] else s[4]
    if kind == "Inverse":
        return np.float32(s[0]) / (np.float32(1.0) + np.float32(s[0]) * np.float32(s[1]) * np.float32(t))
    raise NotImplementedError(kind)


class SgdOpt:
    def __init__(self, step_size=0.01, momentum=("Update", 0.9), l2_reg_coef=0.0):
        self.step_size = np.float32(step_size)
        self.kind, self.mu = (momentum, 0.0) if isinstance(momentum, str) else momentum
        self.mu = np.float32(self.mu)
        self.l2 = np.float32(l2_reg_coef)
        self.iter_counter = 0

    def begin(self, op):
        if self.kind == "UpdateNesterov":
            op.update_params(self.mu)
        op.reset()

    def step(self, op, defer_reapply=False):
        """`defer_reapply`: leave out the Nesterov look-ahead that the reference applies at the very end of an iteration,
        after the checkpoint block (new.rs:623-633); the caller then runs reapply()."""
        step, mu = float(self.step_size), float(self.mu)
        op.regularize(float(self.l2))
        if self.kind == "UpdateNesterov" and self.iter_counter > 0:
            op.update_params(-mu)
        self.iter_counter += 1
        if self.kind == "Zero":
            op.accumulate_grads(-step, 0.0)
        elif self.kind in ("Update", "UpdateNesterov"):
            op.accumulate_grads(-step, mu)
        else:
            op.accumulate_grads(1.0, mu)
        if self.kind in ("Zero", "Update", "UpdateNesterov"):
            op.update_params(1.0)
        elif self.kind == "Gradient":
            op.update_params(-step)
        else:
            op.update_params2(-step, float(np.float32(-step) * self.mu))
        op.reset()
        if self.kind == "UpdateNesterov" and not defer_reapply:
            op.update_params(mu)

    def reapply(self, op):
        if self.kind == "UpdateNesterov":
            op.update_params(float(self.mu))


class SgdOptimization:
    """The minibatch block of the second-generation optimizer, src/opt_new.rs:279-325: per batch (per-sample weights
    1.0) forward -> backward(batch, 1.0) -> accumulate_loss; when a minibatch is complete
    descend(step_size.at_iter(t) / minibatch_size, l2) -> reset_gradients(momentum) -> t += 1."""

    def __init__(self, minibatch_size, step_size=0.01, momentum=0.9, l2_reg_coef=0.0):
        self.minibatch_size = minibatch_size
        self.step_size, self.momentum, self.l2 = np.float32(step_size), np.float32(momentum), np.float32(l2_reg_coef)
        self.t = 0

    def begin(self, arch):
        arch.reset_gradients(0.0)
        arch.reset_loss()

    def batch(self, arch, frames):
        arch.forward(frames)
        arch.backward_scaled(1.0)
        arch.accumulate_loss()

    def end_minibatch(self, arch):
        descent_scale = float(self.step_size / np.float32(self.minibatch_size))
        arch.descend(descent_scale, float(self.l2))
        arch.reset_gradients(float(self.momentum))
        self.t += 1


def sgd_validate(operator, frames, labels):
    """SgdOpt::validate for one worker, new.rs:641-766: the samples in order, full batches then the remainder, Inference
    phase, per-sample weight 1/num_total_samples; returns (sum of the batches' losses, accuracy).  `frames`: float32
    [num][c][h][w] as the input operator hands them on (after its cast)."""
    num = len(labels)
    correct, loss, b0 = 0, np.float32(0.0), 0
    full = operator.batch
    while b0 < num:
        b = min(full, num - b0)
        x = np.zeros((full,) + frames.shape[1:], np.float32)     # operators are built for the batch capacity
        x[:b] = frames[b0:b0 + b]
        lab = np.zeros((full,), np.int32)
        lab[:b] = labels[b0:b0 + b]
        operator.stage_batch(lab, 0.0)
        operator.weights[:b] = np.float32(1.0) / np.float32(num)  # samples past b carry weight 0: they add nothing
        operator.forward(x, training=False, t=0)
        cats = operator.store_output_categories()
        correct += int((cats[:b] == lab[:b]).sum())
        loss = np.float32(loss + np.float32(operator.store_loss()))
        b0 += b
    return float(loss), correct / num


def sgd_train(opt, operator, frames, labels, minibatch_size, max_iters, checkpoint_iters=0, checkpoint_discard=False,
              valid=None, valid_iters=0):
    """SgdOpt::train for one worker from freshly initialised parameters, new.rs:209-640, without its files: returns the
    rows the reference writes to its trace ((iter, "step"|"valid", loss, error)).  Order restated: begin (Nesterov
    look-ahead, reset) -> per sample stage (weight 1/minibatch), per full batch forward(Training{t}) -> categories ->
    loss -> backward -> accuracy count; per minibatch the update block with iter += 1 inside it -> trace row ->
    every checkpoint_iters: [save_params if Discard] -> validation every valid_iters -> [restore_params] -> Nesterov
    look-ahead re-applied last.  Epochs restart at sample 0; a batch never straddles two epochs here
    (len(frames) % batch == 0)."""
    batch = operator.batch
    assert minibatch_size % batch == 0 and len(frames) % batch == 0
    weight = np.float32(1.0) / np.float32(minibatch_size)
    opt.begin(operator)
    rows = []
    local_counter, elapsed_checkpoint_iters = 0, 0
    mb_loss, mb_correct, mb_total = np.float32(0.0), 0, 0
    while opt.iter_counter < max_iters:
        for b0 in range(0, len(frames), batch):
            if opt.iter_counter >= max_iters:
                break
            lab = labels[b0:b0 + batch].astype(np.int32)
            operator.stage_batch(lab, weight)
            local_counter += batch
            operator.forward(frames[b0:b0 + batch], training=True, t=opt.iter_counter)
            cats = operator.store_output_categories()
            mb_loss = np.float32(mb_loss + np.float32(operator.store_loss()))
            operator.backward()
            mb_correct += int((cats == lab).sum())
            mb_total += batch
            if local_counter % minibatch_size != 0:
                continue
            opt.step(operator, defer_reapply=True)
            it = opt.iter_counter
            rows.append((it, "step", float(mb_loss), 1.0 - mb_correct / mb_total))
            mb_loss, mb_correct, mb_total = np.float32(0.0), 0, 0
            if checkpoint_iters and it % checkpoint_iters == 0:
                elapsed_checkpoint_iters += checkpoint_iters
                if checkpoint_discard:
                    operator.save_params()
                if valid is not None and valid_iters and elapsed_checkpoint_iters % valid_iters == 0:
                    vloss, vacc = sgd_validate(operator, valid[0], valid[1])
                    rows.append((it, "valid", vloss, 1.0 - vacc))
                if checkpoint_discard:
                    operator.restore_params()
            opt.reapply(operator)
    return rows
