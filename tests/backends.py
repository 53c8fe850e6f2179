"""The two backends the golden vectors are replayed against: the CPU oracle and the HIP kernels."""
import numpy as np

import oracle_binding as orc
from golden_cases import DomainError, KernelError, OutOfRange


def _st(st):
    if st == orc.ST_DOMAIN:
        raise DomainError()
    if st == 6:
        raise OutOfRange(st)
    if st != 0:
        raise KernelError(st)


class OracleBackend:
    name = "oracle"

    def ew_binary(self, op, a, b):
        st, r = orc.ew_binary(op, a, b); _st(st); return r

    def ew_binary_sca(self, op, a, s):
        st, r = orc.ew_binary_sca(op, a, s); _st(st); return r

    def ew_unary(self, op, a):
        st, r = orc.ew_unary(op, a); _st(st); return r

    def agg_all(self, op, a):
        st, r = orc.agg_all(op, a); _st(st); return float(r)

    def agg_row(self, op, a):
        st, r = orc.agg_row(op, a); _st(st); return r

    def agg_col(self, op, a):
        st, r = orc.agg_col(op, a); _st(st); return r

    def matmul(self, a, b, ta, tb):
        st, r = orc.matmul(a, b, ta, tb); _st(st); return r

    def syrk(self, a, tl):
        st, r = orc.syrk(a, tl); _st(st); return r

    def solve(self, A, b):
        st, r = orc.solve(A, b); _st(st); return r

    def conv2d(self, x, w, bias, N, C, H, W, Hf, Wf, sh, sw, ph, pw):
        st, r, oh, ow = orc.conv2d(x, w, bias, N, C, H, W, Hf, Wf, sh, sw, ph, pw); _st(st); return r, oh, ow

    def maxpool(self, x, N, C, H, W, ph, pw, sh, sw, padh, padw):
        st, r, oh, ow = orc.maxpool(x, N, C, H, W, ph, pw, sh, sw, padh, padw); _st(st); return r, oh, ow

    def bias_add(self, x, b):
        st, r = orc.bias_add(x, b); _st(st); return r

    def batchnorm(self, x, g, b, m, v, eps):
        st, r = orc.batchnorm(x, g, b, m, v, eps, 0); _st(st); return r

    def softmax(self, x):
        st, r = orc.softmax(x); _st(st); return r

    def avgpool(self, x, N, C, H, W, ph, pw, sh, sw, padh, padw):
        st, r, oh, ow = orc.avgpool(x, N, C, H, W, ph, pw, sh, sw, padh, padw); _st(st); return r, oh, ow

    def relu(self, x):
        st, r = orc.relu(x); _st(st); return r

    def transpose(self, x):
        st, r = orc.transpose(x); _st(st); return r

    def col_bind(self, a, b):
        st, r = orc.col_bind(a, b); _st(st); return r

    def extract_col(self, a, sel):
        st, r = orc.extract_col(a, sel); _st(st); return r

    def affine(self, x, w, b):
        st, mm = orc.matmul(x, w); _st(st)
        if b is None:
            return mm
        return mm + b  # 1 x N (or 1 x 1) bias broadcast over rows


    # DNN training kernels
    def batchnorm_train_forward(self, x, g, b, m, v, eps, mu):
        st, *outs = orc.batchnorm_train_forward(x, g, b, m, v, eps, mu)
        _st(st)
        return outs

    def batchnorm_backward(self, mean, inv_var, x, dout, gamma, eps):
        st, *outs = orc.batchnorm_backward(mean, inv_var, x, dout, gamma)
        _st(st)
        return outs

    def maxpool_backward(self, x, dout, *a):
        st, r = orc.maxpool_backward(x, dout, *a)
        _st(st)
        return r

    def avgpool_backward(self, x, dout, *a):
        st, r = orc.avgpool_backward(x, dout, *a)
        _st(st)
        return r

    def conv2d_backward_data(self, filt, dy, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw):
        st, r = orc.conv2d_backward_data(filt, dy, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw)
        _st(st)
        return r

    def conv2d_backward_filter(self, x, dy, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw):
        st, r = orc.conv2d_backward_filter(x, dy, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw)
        _st(st)
        return r


class HipBackend:
    name = "hip"

    def __init__(self, ctx):
        from daphne_amd import capi, kernels
        self.k, self.capi, self.ctx = kernels, capi, ctx

    def _d(self, a):
        if isinstance(a, np.ndarray) and a.ndim == 2 and a.size and not a.flags.c_contiguous and a.base is not None:
            # a view with a row stride: upload the array it looks into and pass the same view of the device copy
            root = a
            while root.base is not None:
                root = root.base
            if isinstance(root, np.ndarray) and root.ndim == 2 and root.flags.c_contiguous and a.strides[1] == a.itemsize \
                    and a.strides[0] == root.strides[0]:
                off = (a.ctypes.data - root.ctypes.data) // a.itemsize
                r0, c0 = divmod(off, root.shape[1])
                return self.k.DenseMatrix.from_numpy(self.ctx, root).slice(r0, r0 + a.shape[0], c0, c0 + a.shape[1])
        return self.k.DenseMatrix.from_numpy(self.ctx, a)

    def _call(self, fn, *a):
        try:
            return fn(*a)
        except self.capi.DaphneHipDomainError:
            raise DomainError()
        except self.capi.DaphneHipOutOfRange as e:
            raise OutOfRange(str(e))
        except self.capi.DaphneHipError as e:
            raise KernelError(str(e))

    def ew_binary(self, op, a, b):
        return self._call(self.k.ewBinaryMat, op, None, self._d(a), self._d(b), self.ctx).to_numpy()

    def ew_binary_sca(self, op, a, s):
        return self._call(self.k.ewBinaryObjSca, op, None, self._d(a), s, self.ctx).to_numpy()

    def ew_unary(self, op, a):
        return self._call(self.k.ewUnaryMat, op, None, self._d(a), self.ctx).to_numpy()

    def agg_all(self, op, a):
        return float(self._call(self.k.aggAll, op, self._d(a), self.ctx))

    def agg_row(self, op, a):
        return self._call(self.k.aggRow, op, None, self._d(a), self.ctx).to_numpy()

    def agg_col(self, op, a):
        return self._call(self.k.aggCol, op, None, self._d(a), self.ctx).to_numpy()

    def matmul(self, a, b, ta, tb):
        return self._call(self.k.matMul, None, self._d(a), self._d(b), ta, tb, self.ctx).to_numpy()

    def syrk(self, a, tl):
        return self._call(self.k.syrk, None, self._d(a), tl, self.ctx).to_numpy()

    def solve(self, A, b):
        return self._call(self.k.solve, None, self._d(A), self._d(b), self.ctx).to_numpy()

    def conv2d(self, x, w, bias, N, C, H, W, Hf, Wf, sh, sw, ph, pw):
        r, oh, ow = self._call(self.k.conv2dForward, None, self._d(x), self._d(w),
                               self._d(bias) if bias is not None else None, N, C, H, W, Hf, Wf, sh, sw, ph, pw, self.ctx)
        return r.to_numpy(), oh, ow

    def maxpool(self, x, N, C, H, W, ph, pw, sh, sw, padh, padw):
        r, oh, ow = self._call(self.k.maxPoolForward, None, self._d(x), N, C, H, W, ph, pw, sh, sw, padh, padw, self.ctx)
        return r.to_numpy(), oh, ow

    def avgpool(self, x, N, C, H, W, ph, pw, sh, sw, padh, padw):
        r, oh, ow = self._call(self.k.avgPoolForward, None, self._d(x), N, C, H, W, ph, pw, sh, sw, padh, padw, self.ctx)
        return r.to_numpy(), oh, ow

    def relu(self, x):
        return self._call(self.k.reluForward, None, self._d(x), self.ctx).to_numpy()

    def transpose(self, x):
        return self._call(self.k.transpose, None, self._d(x), self.ctx).to_numpy()

    def col_bind(self, a, b):
        return self._call(self.k.colBind, None, self._d(a), self._d(b), self.ctx).to_numpy()

    def extract_col(self, a, sel):
        return self._call(self.k.extractCol, None, self._d(a), self._d(np.ascontiguousarray(sel, dtype=np.int64)),
                          self.ctx).to_numpy()

    def bias_add(self, x, b):
        return self._call(self.k.biasAdd, None, self._d(x), self._d(b), self.ctx).to_numpy()

    def batchnorm(self, x, g, b, m, v, eps):
        return self._call(self.k.batchNormInferenceForward, None, self._d(x), self._d(g), self._d(b), self._d(m),
                          self._d(v), eps, self.ctx).to_numpy()

    def softmax(self, x):
        return self._call(self.k.softmax, None, self._d(x), self.ctx).to_numpy()

    def affine(self, x, w, b):
        return self._call(self.k.affineForward, None, self._d(x), self._d(w), self._d(b) if b is not None else None,
                          self.ctx).to_numpy()

    # DNN training kernels
    def batchnorm_train_forward(self, x, g, b, m, v, eps, mu):
        outs = self._call(self.k.batchNorm2DTrainForward, self._d(x), self._d(g), self._d(b), self._d(m), self._d(v), eps, mu, self.ctx)
        return [o.to_numpy() for o in outs]

    def batchnorm_backward(self, mean, inv_var, x, dout, gamma, eps):
        outs = self._call(self.k.batchNorm2DBackward, self._d(mean), self._d(inv_var), self._d(x), self._d(dout), self._d(gamma), eps,
                          self.ctx)
        return [o.to_numpy() for o in outs]

    def maxpool_backward(self, x, dout, *a):
        return self._call(self.k.maxPoolBackward, None, self._d(x), self._d(dout), *a, self.ctx).to_numpy()

    def avgpool_backward(self, x, dout, *a):
        return self._call(self.k.avgPoolBackward, None, self._d(x), self._d(dout), *a, self.ctx).to_numpy()

    def conv2d_backward_data(self, filt, dy, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw):
        return self._call(self.k.conv2DBackwardData, self._d(filt), self._d(dy), sh, sw, ph, pw, N, C, H, W, F, C, Hf, Wf, None,
                          self.ctx).to_numpy()

    def conv2d_backward_filter(self, x, dy, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw):
        return self._call(self.k.conv2DBackwardFilter, None, self._d(x), self._d(dy), sh, sw, ph, pw, N, C, H, W, F, C, Hf, Wf,
                          self.ctx).to_numpy()
