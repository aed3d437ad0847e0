"""Allocation-free driver of the network body on the C ABI: ``outer`` x (step, LayerNorm)
forward, then the same chain backward, on preallocated buffers.

This is what a training loop that owns its buffers (or a captured HIP graph) calls; the
autograd ops in ``backend_cuda``/``layernorm`` do the same launches with torch-managed
memory.  Order of operations: gridnet/scripts/train_mnist.py:62-64.

``fused=True`` runs the same chain through the entry points that fold the LayerNorm into the
step kernels: a step reads the raw output of the step before it and normalises it while
loading, so the LayerNorm costs no pass over the activations of its own (one, for the final
output).  Same results within rounding; fp32, ``normalize=False``, ``inner >= 1`` only.

With ``fused=True`` and a problem it covers (float32, 8^3 blocks, up to 8 inner iterations) the
backward of a chain can go through ``gridnet_hip_chain_backward``: the backward hands what
crosses a block boundary from step to step instead of finishing every dx (one kernel per step
instead of two).  Same results to rounding.  ``chain=None`` (the default) takes it where the
two-kernel backward would have to deal its cross-block part by block face (rows of other than 16,
32, 64 or 128 cells); where that part goes by whole rows the two kernels are the faster pair
(64^3 grid, batch 32, 12 steps: 3.12 against 3.19 ms per training step).  ``True``: wherever the
library supports it; ``False``: never (nor the one launch below).

Where the whole grid fits the GPU at once (every block a resident workgroup: a 64^3 grid on an
MI355X) and the steps share one parameter set, the chain backward is ONE launch
(``gridnet_hip_chain_backward_all``, ``chain_all=None`` picks it when the grid fills the chip,
``True`` wherever the library supports it, ``False`` never): the workgroups keep their blocks,
weights and gradient accumulators from step to step and signal each other through memory.  Its
waits are bounded; ``chain_all_status()`` (which synchronises) tells whether one ran out, in which
case ``backward`` must be repeated with ``chain_all`` off -- ``backward_checked`` does both.

``weight``, ``bias`` and ``scale`` may each be a list of ``outer`` tensors: one parameter set
per outer step (the reference's ``--separate_params``, gridnet/scripts/train_imagenet.py:54-58).
``backward`` then returns lists of gradients for them, one entry per step.

``outer_residual=True`` is the other shape of the loop, ``n = norm(h); h = h + (net(n) - n)``
(gridnet/scripts/train_imagenet.py:81-83), through the fused entry points made for it
(``fused=True`` only).
"""

import torch

from . import native as _n


class BodyRunner:
    def __init__(self, weight, bias, scale, gamma, beta, batch: int, inner: int, outer: int,
                 block_size: int, activation: str = "leaky_relu", normalize: bool = False,
                 eps: float = 1e-5, ln_eps: float = 1e-5, backward: bool = True,
                 fused: bool = False, outer_residual: bool = False, chain=None,
                 chain_all=None):
        self.separate = isinstance(weight, (list, tuple))
        if self.separate:
            if not (len(weight) == len(bias) == len(scale) == outer):
                raise ValueError("separate parameters: one weight, bias and scale per outer step")
            self.ws, self.bs_, self.rs = list(weight), list(bias), list(scale)
        else:
            self.ws, self.bs_, self.rs = [weight] * max(outer, 1), [bias] * max(outer, 1), [scale] * max(outer, 1)
        weight, bias, scale = self.ws[0], self.bs_[0], self.rs[0]
        self.w, self.b, self.r, self.gamma, self.beta = weight, bias, scale, gamma, beta
        self.B, (self.M, self.N, self.K) = batch, bias.shape
        if outer < 1:
            raise ValueError(f"outer must be at least 1, got {outer}")
        self.inner, self.outer, self.bs = inner, outer, block_size
        self.act = _n.activation_id(activation)
        self.normalize, self.eps, self.ln_eps = int(normalize), eps, ln_eps
        self.dt = _n.dtype_id(weight)
        dev, dtype = weight.device, weight.dtype
        n = bias.numel()
        self.n = n
        shape = (batch, self.M, self.N, self.K)
        keep = outer if backward else 1
        if outer_residual and not fused:
            raise RuntimeError("outer_residual runs through the fused entry points only (fused=True)")
        # h[j]: input of outer step j (h[outer] = result); s[j]: its output before the norm.
        # What a mode never touches is not allocated: the fused chain keeps the raw outputs s[*]
        # and one h (the final result; forward only, a second buffer to alternate with), the
        # residual chain every h and two s (free buffers for its backward).
        n_h, n_s = keep + 1, keep
        if fused and not outer_residual:
            n_h = 1 if backward else 2
        if fused and outer_residual:
            n_s = 2 if backward else 1
        self.h = [torch.empty(shape, device=dev, dtype=dtype) for _ in range(n_h)]
        # one allocation: the one-launch chain backward takes the raw outputs as [outer, B, M, N, K]
        self.s_all = torch.empty((n_s,) + shape, device=dev, dtype=dtype)
        self.s = list(self.s_all)
        self.mean = torch.empty(keep, batch, device=dev, dtype=dtype)
        self.rstd = torch.empty(keep, batch, device=dev, dtype=dtype)
        self.ln_ws_bytes = _n.lib.gridnet_hip_layernorm_workspace_bytes(self.dt, batch, n)
        self.ln_ws = _n.workspace(self.ln_ws_bytes, dev)
        self.has_backward = backward
        if backward:
            self.ga = torch.empty(shape, device=dev, dtype=dtype)
            self.gb = torch.empty(shape, device=dev, dtype=dtype)
            # one gradient set per parameter set.  The entry points either overwrite all parameter
            # gradients of a call or accumulate into all of them, the LayerNorm's (shared by the
            # steps) included: with separate parameters the last step's call overwrites, the
            # others accumulate into buffers that backward() zero-fills first
            n_sets = outer if self.separate else 1
            self.dw_all = torch.empty((n_sets,) + tuple(weight.shape), device=dev, dtype=dtype)
            self.db_all = torch.empty((n_sets,) + tuple(bias.shape), device=dev, dtype=dtype)
            self.dr_all = torch.empty((n_sets,) + tuple(bias.shape), device=dev, dtype=dtype)
            self.dgamma = torch.empty_like(bias)
            self.dbeta = torch.empty_like(bias)
            self.bw_ws_bytes = _n.lib.gridnet_hip_backward_workspace_bytes(
                self.dt, batch, self.M, self.N, self.K, inner, block_size, self.normalize)
            self.bw_ws = _n.workspace(self.bw_ws_bytes, dev)
        self.on_launch = None  # optional hook(name, phase) for per-kernel timing
        self.fused = fused
        self.outer_residual = outer_residual
        if fused:
            if weight.dtype != torch.float32 or normalize or inner < 1:
                raise RuntimeError("the fused body covers float32, normalize=False, inner >= 1")
            self.stats = torch.empty(max(keep, 2), batch, 2, device=dev, dtype=dtype)
            self.fw_ws_bytes = _n.lib.gridnet_hip_fused_workspace_bytes(
                batch, self.M, self.N, self.K, inner, block_size, 0)
            self.fw_ws = _n.workspace(self.fw_ws_bytes, dev)
            if outer_residual:  # statistics of h_0 .. h_outer, and a LayerNorm output nobody reads
                self.stats = torch.empty(keep + 1, batch, 2, device=dev, dtype=dtype)
                self.unused = torch.empty(shape, device=dev, dtype=dtype)
            if backward:
                self.sums = torch.empty(keep, batch, 2, device=dev, dtype=dtype)
                self.fb_ws_bytes = _n.lib.gridnet_hip_fused_workspace_bytes(
                    batch, self.M, self.N, self.K, inner, block_size, 1)
                self.fb_ws = _n.workspace(self.fb_ws_bytes, dev)
        chain_ok = bool(chain is not False and fused and backward and not outer_residual and
                        _n.lib.gridnet_hip_chain_supported(self.dt, inner, block_size, self.normalize))
        rows = self.K in (16, 32, 64, 128)  # what the row-wise cross-block kernel takes
        self.chain = chain_ok and (chain is True or not rows)
        if self.chain:
            # two buffers that the backward calls of neighbouring steps hand their cross-block
            # values over in
            nfl = _n.lib.gridnet_hip_chain_halo_floats(batch, self.M, self.N, self.K, block_size)
            self.halo = [torch.empty(nfl, device=dev, dtype=dtype) for _ in range(2 if outer > 1 else 0)]
        self.chain_all = False
        if chain_ok and not self.separate and chain_all is not False and \
                _n.lib.gridnet_hip_chain_all_supported(self.dt, batch, self.M, self.N, self.K, inner, outer,
                                                       block_size, self.normalize):
            nblk = (self.M // 8) * (self.N // 8) * (self.K // 8)
            cus = torch.cuda.get_device_properties(dev).multi_processor_count
            self.chain_all = bool(chain_all) or nblk >= cus
        if self.chain_all:
            self.ca_ws_bytes = _n.lib.gridnet_hip_chain_all_workspace_bytes(
                batch, self.M, self.N, self.K, inner, outer, block_size)
            self.ca_ws = _n.workspace(self.ca_ws_bytes, dev)

    def _params(self, j):
        """Device pointers of the parameter set of outer step j."""
        return self.ws[j].data_ptr(), self.bs_[j].data_ptr(), self.rs[j].data_ptr()

    def _grads(self, j):
        """Device pointers of the gradient buffers that outer step j accumulates into."""
        k = j if self.separate else 0
        return self.dw_all[k].data_ptr(), self.db_all[k].data_ptr(), self.dr_all[k].data_ptr()

    def _param_grads(self):
        if self.separate:
            return list(self.dw_all), list(self.db_all), list(self.dr_all)
        return self.dw_all[0], self.db_all[0], self.dr_all[0]

    def _zero_separate_grads(self):
        if self.separate and self.outer > 1:
            self.dw_all[:-1].zero_()
            self.db_all[:-1].zero_()
            self.dr_all[:-1].zero_()

    def _mark(self, name, phase):
        if self.on_launch is not None:
            self.on_launch(name, phase)

    def step_forward(self, x, y, stream, j=0):
        self._mark("step_fwd", 0)
        _n.check(_n.lib.gridnet_hip_forward(
            self.dt, *self._params(j), x.data_ptr(),
            y.data_ptr(), self.B, self.M, self.N, self.K, self.inner, self.bs, self.eps,
            self.normalize, self.act, stream))
        self._mark("step_fwd", 1)

    def norm_forward(self, x, y, j, stream):
        self._mark("ln_fwd", 0)
        _n.check(_n.lib.gridnet_hip_layernorm_forward(
            self.dt, x.data_ptr(), self.gamma.data_ptr(), self.beta.data_ptr(), y.data_ptr(),
            self.mean[j].data_ptr(), self.rstd[j].data_ptr(), self.B, self.n, self.ln_eps,
            self.ln_ws.data_ptr(), self.ln_ws_bytes, stream))
        self._mark("ln_fwd", 1)

    # ---- the fused chain: s[j] = raw output of step j, stats[j] = its LayerNorm statistics ----
    def _fused_forward(self, x0):
        stream = _n.current_stream(self.w)
        keep = self.has_backward
        self.x0 = x0
        x, x_stats = x0, None
        for j in range(self.outer):
            # forward only: nothing is kept, two raw buffers and two statistics rows alternate
            y = self.s[j] if keep else (self.s[0], self.h[1])[j % 2]
            y_stats = self.stats[j if keep else j % 2]
            self._mark("step_fwd", 0)
            # every other step walks the blocks in reverse: what the step before touched last is
            # what this one needs first (it matters where a step's working set exceeds the
            # last-level cache, a 128^3 grid; the results are the same bits)
            _n.check(_n.lib.gridnet_hip_fused_forward_flags(
                self.dt, *self._params(j),
                self.gamma.data_ptr(), self.beta.data_ptr(), x.data_ptr(),
                x_stats.data_ptr() if x_stats is not None else None, y.data_ptr(),
                y_stats.data_ptr(), self.B, self.M, self.N, self.K, self.inner, self.bs,
                self.ln_eps, self.act, _n.FUSED_WALK_REVERSE if j & 1 else 0,
                self.fw_ws.data_ptr(), self.fw_ws_bytes, stream))
            self._mark("step_fwd", 1)
            x, x_stats = y, y_stats
        out = self.h[0]
        self._mark("ln_fwd", 0)
        _n.check(_n.lib.gridnet_hip_layernorm_apply(
            self.dt, x.data_ptr(), x_stats.data_ptr(), self.gamma.data_ptr(), self.beta.data_ptr(),
            out.data_ptr(), self.B, self.n, stream))
        self._mark("ln_fwd", 1)
        return out

    def _residual_forward(self, x0):
        """h = h + (net(norm(h)) - norm(h)), ``outer`` times; returns the last h as it is."""
        stream = _n.current_stream(self.w)
        keep = self.has_backward
        self.x0 = x0
        # statistics of the first input: the LayerNorm entry point's, its output unused
        self.norm_forward(x0, self.unused, 0, stream)
        self.stats[0, :, 0].copy_(self.mean[0])
        self.stats[0, :, 1].copy_(self.rstd[0])
        h, stats = x0, self.stats[0]
        for j in range(self.outer):
            # h[j + 1] and stats[j + 1] are kept for the backward; forward only, two of each alternate
            out = self.h[j + 1] if keep else (self.s[0], self.h[1])[j % 2]
            out_stats = self.stats[j + 1 if keep else (j + 1) % 2]
            self._mark("step_fwd", 0)
            _n.check(_n.lib.gridnet_hip_fused_forward_flags(
                self.dt, *self._params(j),
                self.gamma.data_ptr(), self.beta.data_ptr(), h.data_ptr(), stats.data_ptr(),
                out.data_ptr(), out_stats.data_ptr(), self.B, self.M, self.N, self.K, self.inner,
                self.bs, self.ln_eps, self.act,
                _n.FUSED_RESIDUAL | (_n.FUSED_WALK_REVERSE if j & 1 else 0),
                self.fw_ws.data_ptr(), self.fw_ws_bytes, stream))
            self._mark("step_fwd", 1)
            h, stats = out, out_stats
        return h

    def _residual_backward(self, grad_out):
        """With G_k the gradient with respect to h_k (G_outer = grad_out): step j forms G_{j+1}
        from G_{j+2} and the dn of step j+1 as it loads them, and leaves dn_j; the chain's input
        gradient is G_1 + LayerNorm'(dn_0)."""
        stream = _n.current_stream(self.w)
        last = self.outer - 1
        dn = [self.ga, self.gb]       # dn_j alternates between the two
        gbuf = [self.s[0], self.s[-1]]  # G_k for 0 < k < outer: the s buffers are free in this shape

        def grad_wrt(k):  # G_k
            return grad_out if k == self.outer else gbuf[k % 2]

        for j in reversed(range(self.outer)):
            given = j == last
            x = self.h[j] if j else self.x0
            self._mark("step_bwd", 0)
            _n.check(_n.lib.gridnet_hip_fused_backward_residual(
                self.dt, *self._params(j),
                self.gamma.data_ptr(), self.beta.data_ptr(), x.data_ptr(), self.stats[j].data_ptr(),
                (grad_out if given else dn[(j + 1) % 2]).data_ptr(),
                None if given else self.h[j + 1].data_ptr(),
                None if given else self.stats[j + 1].data_ptr(),
                None if given else self.sums[j + 1].data_ptr(),
                None if given else grad_wrt(j + 2).data_ptr(),
                None if given else grad_wrt(j + 1).data_ptr(),
                *self._grads(j), self.dgamma.data_ptr(),
                self.dbeta.data_ptr(), dn[j % 2].data_ptr(), self.sums[j].data_ptr(),
                self.B, self.M, self.N, self.K, self.inner, self.bs, self.act,
                _n.OVERWRITE_PARAMS if given else 0, self.fb_ws.data_ptr(), self.fb_ws_bytes, stream))
            self._mark("step_bwd", 1)
        # the LayerNorm in front of the first step: dx0 = G_1 + LayerNorm'(dn_0), with its dgamma, dbeta
        self._mark("ln_bwd", 0)
        _n.check(_n.lib.gridnet_hip_layernorm_backward(
            self.dt, dn[0].data_ptr(), self.x0.data_ptr(), self.gamma.data_ptr(),
            self.mean[0].data_ptr(), self.rstd[0].data_ptr(), dn[1].data_ptr(),
            self.dgamma.data_ptr(), self.dbeta.data_ptr(), self.B, self.n, 0,
            self.ln_ws.data_ptr(), self.ln_ws_bytes, stream))
        self._mark("ln_bwd", 1)
        torch.add(dn[1], grad_wrt(1), out=dn[1])
        return (*self._param_grads(), self.dgamma, self.dbeta, dn[1])

    def chain_all_status(self) -> int:
        """Synchronises.  Non-zero: a bounded wait of the last one-launch backward ran out and its
        results are invalid."""
        if not self.chain_all:
            return 0
        return int(self.ca_ws[:4].view(torch.int32).item())

    def backward_checked(self, grad_out):
        """``backward``; should the one-launch chain report that it gave up, the one-launch path is
        switched off for this runner and the backward repeated launch by launch.  Synchronises."""
        out = self.backward(grad_out)
        if self.chain_all and self.chain_all_status() != 0:
            self.chain_all = False
            out = self.backward(grad_out)
        return out

    def _chain_all_backward(self, grad_out):
        stream = _n.current_stream(self.w)
        self._mark("step_bwd", 0)
        _n.check(_n.lib.gridnet_hip_chain_backward_all(
            self.dt, *self._params(0), self.gamma.data_ptr(), self.beta.data_ptr(), self.x0.data_ptr(),
            self.s_all.data_ptr(), self.stats.data_ptr(), grad_out.data_ptr(),
            *self._grads(0), self.dgamma.data_ptr(), self.dbeta.data_ptr(), self.ga.data_ptr(),
            self.B, self.M, self.N, self.K, self.inner, self.outer, self.bs, self.act,
            _n.OVERWRITE_PARAMS, self.ca_ws.data_ptr(), self.ca_ws_bytes, stream))
        self._mark("step_bwd", 1)
        return (*self._param_grads(), self.dgamma, self.dbeta, self.ga)

    def _fused_backward(self, grad_out):
        if self.chain_all:
            return self._chain_all_backward(grad_out)
        stream = _n.current_stream(self.w)
        last = self.outer - 1
        self._mark("ln_bwd", 0)
        _n.check(_n.lib.gridnet_hip_layernorm_backward_sums(
            self.dt, grad_out.data_ptr(), self.s[last].data_ptr(), self.stats[last].data_ptr(),
            self.gamma.data_ptr(), self.sums[last].data_ptr(), self.B, self.n,
            self.ln_ws.data_ptr(), self.ln_ws_bytes, stream))
        self._mark("ln_bwd", 1)
        g = grad_out
        for j in reversed(range(self.outer)):
            x = self.s[j - 1] if j else self.x0
            dst = self.ga if g is not self.ga else self.gb
            self._mark("step_bwd", 0)
            if self.chain:
                # dx of every step but the first stays unfinished: what crosses a block boundary
                # travels in halo[j % 2] to the call for step j - 1
                _n.check(_n.lib.gridnet_hip_chain_backward(
                    self.dt, *self._params(j),
                    self.gamma.data_ptr(), self.beta.data_ptr(), x.data_ptr(),
                    self.stats[j - 1].data_ptr() if j else None, g.data_ptr(), self.s[j].data_ptr(),
                    self.stats[j].data_ptr(), self.sums[j].data_ptr(),
                    None if j == last else self.halo[(j + 1) % 2].data_ptr(),
                    self.halo[j % 2].data_ptr() if j else None,
                    *self._grads(j), self.dgamma.data_ptr(), self.dbeta.data_ptr(), dst.data_ptr(),
                    self.sums[j - 1].data_ptr() if j else None, self.B, self.M, self.N, self.K,
                    self.inner, self.bs, self.act, _n.OVERWRITE_PARAMS if j == last else 0,
                    self.fb_ws.data_ptr(), self.fb_ws_bytes, stream))
                self._mark("step_bwd", 1)
                g = dst
                continue
            _n.check(_n.lib.gridnet_hip_fused_backward(
                self.dt, *self._params(j),
                self.gamma.data_ptr(), self.beta.data_ptr(), x.data_ptr(),
                self.stats[j - 1].data_ptr() if j else None, g.data_ptr(), self.s[j].data_ptr(),
                self.stats[j].data_ptr(), self.sums[j].data_ptr(), *self._grads(j), self.dgamma.data_ptr(),
                self.dbeta.data_ptr(), dst.data_ptr(), self.sums[j - 1].data_ptr() if j else None,
                self.B, self.M, self.N, self.K, self.inner, self.bs, self.act,
                _n.OVERWRITE_PARAMS if j == last else 0, self.fb_ws.data_ptr(), self.fb_ws_bytes,
                stream))
            self._mark("step_bwd", 1)
            g = dst
        return (*self._param_grads(), self.dgamma, self.dbeta, g)

    def forward(self, x0):
        """Returns the buffer holding the result (valid until the next call)."""
        if self.outer_residual:
            return self._residual_forward(x0)
        if self.fused:
            return self._fused_forward(x0)
        stream = _n.current_stream(self.w)
        self.x0 = x0  # read in place (and again by backward): the caller keeps it unchanged
        if self.has_backward:
            for j in range(self.outer):
                self.step_forward(self.h[j] if j else x0, self.s[j], stream, j)
                self.norm_forward(self.s[j], self.h[j + 1], j, stream)
            return self.h[self.outer]
        for j in range(self.outer):  # forward only: ping-pong, nothing is kept
            self.step_forward(self.h[j % 2] if j else x0, self.s[0], stream, j)
            self.norm_forward(self.s[0], self.h[(j + 1) % 2], 0, stream)
        return self.h[self.outer % 2]

    def backward(self, grad_out):
        """Backward of the last ``forward``.  Returns (dweight, dbias, dscale, dgamma, dbeta, dx0);
        parameter gradients are summed over the outer steps (shared parameters)."""
        assert self.has_backward
        self._zero_separate_grads()
        if self.outer_residual:
            return self._residual_backward(grad_out)
        if self.fused:
            return self._fused_backward(grad_out)
        stream = _n.current_stream(self.w)
        g = grad_out
        for j in reversed(range(self.outer)):
            flags = _n.OVERWRITE_PARAMS if j == self.outer - 1 else 0
            self._mark("ln_bwd", 0)
            _n.check(_n.lib.gridnet_hip_layernorm_backward(
                self.dt, g.data_ptr(), self.s[j].data_ptr(), self.gamma.data_ptr(),
                self.mean[j].data_ptr(), self.rstd[j].data_ptr(), self.ga.data_ptr(),
                self.dgamma.data_ptr(), self.dbeta.data_ptr(), self.B, self.n, flags,
                self.ln_ws.data_ptr(), self.ln_ws_bytes, stream))
            self._mark("ln_bwd", 1)
            self._mark("step_bwd", 0)
            # dx is fully written every time; parameter gradients are written by the first
            # call and accumulated into by the later ones (parameters are shared)
            _n.check(_n.lib.gridnet_hip_backward(
                self.dt, *self._params(j),
                (self.h[j] if j else self.x0).data_ptr(), self.ga.data_ptr(), *self._grads(j),
                self.gb.data_ptr(), self.B, self.M, self.N, self.K, self.inner,
                self.bs, self.eps, self.normalize, self.act, flags | _n.OVERWRITE_DX,
                self.bw_ws.data_ptr(), self.bw_ws_bytes, stream))
            self._mark("step_bwd", 1)
            g = self.gb
        return (*self._param_grads(), self.dgamma, self.dbeta, self.gb)
