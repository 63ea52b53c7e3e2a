"""Host-side mirror of the engine's tensor operators that call the matmul path.

``Tensor`` is a shape plus a device buffer; its methods derive the raw-pointer argument
lists exactly as the reference's ``VTensor`` methods do and issue the same sequence of
``VMath`` calls:

* ``matmul`` / ``matmul_backprop``   -- api_objects/vtensor.cpp:1282-1375
* ``add`` / ``add_backprop``         -- api_objects/vtensor.cpp:3395-3485
* ``activate`` / ``activate_backprop`` -- api_objects/vtensor.cpp:5674-5718
* ``mh_attention`` / ``mh_attention_backprop`` -- api_objects/vtensor.cpp:2978-3227
* ``rnn`` / ``rnn_backprop`` (module level)  -- api_objects/vtensor.cpp:2350-2522, 2524-2717

Shape errors raise ``KaiError`` with the reference's codes (VERR_BAD_SHAPE_TENSOR = 10003).
The graph, autograd queue and tracer of the engine are not rebuilt: backprop methods
return the gradients instead of registering them in a queue.
"""
import numpy as np

from . import kai
from .kai import ACT, DeviceBuffer, KaiError, VMath

VERR_BAD_SHAPE_TENSOR = 10003
VERR_UNDEFINED = 2


def _total(shape):
    n = 1
    for s in shape:
        n *= int(s)
    return n


class Tensor:
    """A float32 device tensor: ``shape`` and a ``DeviceBuffer`` (reference: VTensor + VTensorData)."""

    def __init__(self, shape, device=0, buf=None):
        self.shape = tuple(int(s) for s in shape)
        self.device = device
        self.buf = buf if buf is not None else DeviceBuffer(max(_total(self.shape), 1) * 4, device)
        self.saved = {}

    @classmethod
    def from_numpy(cls, a, device=0):
        a = np.ascontiguousarray(a, dtype=np.float32)
        return cls(a.shape, device, DeviceBuffer.from_numpy(a, device))

    def numpy(self):
        return self.buf.to_numpy(self.shape, np.float32)

    @property
    def ptr(self):
        return self.buf.ptr

    def total_size(self):
        return _total(self.shape)

    # ---- matmul: vtensor.cpp:1282-1335 ------------------------------------------------------------
    def matmul(self, w):
        x = self
        if len(x.shape) < 2:
            raise KaiError(VERR_BAD_SHAPE_TENSOR, "matmul")
        if len(w.shape) != 2:
            raise KaiError(VERR_BAD_SHAPE_TENSOR, "matmul")
        yvec, xvec = w.shape
        ndat = x.total_size() // xvec
        yshape = list(x.shape)
        while True:
            yshape = yshape[:-1]
            t = _total(yshape)
            if t == ndat:
                break
            if t < ndat:
                raise KaiError(VERR_UNDEFINED, "matmul: input cannot be split into rows of the weight's width")
        yshape.append(yvec)
        y = Tensor(yshape, x.device)
        VMath.matmul(x.device, y.ptr, w.ptr, x.ptr, yvec, ndat, xvec, False)
        y.saved = {"op": "matmul", "x": x, "w": w}
        return y

    # vtensor.cpp:1337-1375
    def matmul_backprop(self, ygrad, need_x=True, need_w=True):
        x, w = self.saved["x"], self.saved["w"]
        yvec, xvec = w.shape
        ndat = x.total_size() // xvec
        xgrad = wgrad = None
        if need_x:
            xgrad = Tensor(x.shape, x.device)
            VMath.matmul_backward_x(x.device, xgrad.ptr, ygrad.ptr, w.ptr, yvec, ndat, xvec, False)
        if need_w:
            wgrad = Tensor(w.shape, x.device)
            VMath.matmul_backward_w(x.device, wgrad.ptr, ygrad.ptr, x.ptr, yvec, ndat, xvec, False)
        return xgrad, wgrad

    # ---- add (bias form): vtensor.cpp:3395-3436 -----------------------------------------------------
    def add(self, b):
        a = self
        if a.shape != b.shape and a.total_size() % b.total_size() != 0:
            raise KaiError(VERR_BAD_SHAPE_TENSOR, "add")
        if a.shape == b.shape:
            raise NotImplementedError("same-shape add is VMath::add, outside the matmul path")
        ndat = a.total_size()
        ncol = b.total_size()
        nrow = ndat // ncol
        y = Tensor(a.shape, a.device)
        VMath.add_bias(a.device, y.ptr, a.ptr, b.ptr, nrow, ncol)
        y.saved = {"op": "add", "a": a, "b": b}
        return y

    # vtensor.cpp:3438-3485 (bias branch): the gradient of `a` is ygrad itself
    def add_backprop(self, ygrad):
        a, b = self.saved["a"], self.saved["b"]
        ndat = a.total_size()
        ncol = b.shape[-1]
        nrow = ndat // ncol
        bgrad = Tensor(b.shape, a.device)
        VMath.add_bias_backward_b(a.device, bgrad.ptr, ygrad.ptr, nrow, ncol, False)
        return ygrad, bgrad

    # ---- activate: vtensor.cpp:5674-5695 ---------------------------------------------------------------
    def activate(self, actfunc, leaky_alpha=None):
        x = self
        ncol = x.shape[-1]
        nrow = x.total_size() // ncol
        code = ACT[actfunc] if isinstance(actfunc, str) else int(actfunc)
        h = kai.hyper(leaky_alpha, x.device)
        y = Tensor(x.shape, x.device)
        VMath.activate(x.device, y.ptr, x.ptr, nrow, ncol, code, h)
        y.saved = {"op": "activate", "x": x, "actfunc": code, "leaky_alpha": h}
        return y

    # vtensor.cpp:5697-5718
    def activate_backprop(self, ygrad):
        x = self.saved["x"]
        ncol = self.shape[-1]
        nrow = self.total_size() // ncol
        xgrad = Tensor(x.shape, x.device)
        VMath.activate_backward(x.device, xgrad.ptr, ygrad.ptr, x.ptr, nrow, ncol, self.saved["actfunc"],
                                self.saved["leaky_alpha"])
        return xgrad

    # ---- mh_attention: vtensor.cpp:2978-3052 ----------------------------------------------------------
    def mh_attention(self, key, query, value, Kw, Kb, Qw, Qb, Vw, Vb, Ow, Ob, head_cnt, mask=False, coef=None,
                     fused=False):
        """``fused=False`` issues the reference's calls one by one; ``fused=True`` replaces the middle of the block
        (mult_on_heads, mask, softmax_direct_on_axis, mix_values) by one kai_attention_forward_train."""
        x = self
        if len(x.shape) != 3 or x.shape[2] % head_cnt != 0:
            raise KaiError(VERR_BAD_SHAPE_TENSOR, "mh_attention")
        if x.shape != key.shape or x.shape != query.shape or x.shape != value.shape:
            raise KaiError(VERR_BAD_SHAPE_TENSOR, "mh_attention")
        nbat, ntimes, nvec = x.shape
        nhead = head_cnt
        npiece = nvec // nhead
        for w in (Kw, Qw, Vw):
            if w.shape != (nvec, nvec):
                raise KaiError(VERR_BAD_SHAPE_TENSOR, "mh_attention")
        if coef is None:
            coef = 1.0 / np.sqrt(nvec / nhead)   # api_objects/vmodule.cpp:1805
        hcoef = kai.hyper(coef, x.device)
        dev = x.device
        y = Tensor(x.shape, dev)
        K = Tensor((nbat, ntimes, nvec), dev)
        Q = Tensor((nbat, ntimes, nvec), dev)
        V = Tensor((nbat, ntimes, nvec), dev)
        probs = Tensor((nbat, ntimes, ntimes, nhead), dev)
        mixed = Tensor(x.shape, dev)
        n = nbat * ntimes
        VMath.matmul(dev, K.ptr, Kw.ptr, key.ptr, nvec, n, nvec, False)
        VMath.matmul(dev, Q.ptr, Qw.ptr, query.ptr, nvec, n, nvec, False)
        VMath.matmul(dev, V.ptr, Vw.ptr, value.ptr, nvec, n, nvec, False)
        VMath.add_bias(dev, K.ptr, K.ptr, Kb.ptr, n, nvec)
        VMath.add_bias(dev, Q.ptr, Q.ptr, Qb.ptr, n, nvec)
        VMath.add_bias(dev, V.ptr, V.ptr, Vb.ptr, n, nvec)
        if fused:
            VMath.attention_forward_train(dev, mixed.ptr, probs.ptr, Q.ptr, K.ptr, V.ptr, nbat, ntimes, nvec, nhead,
                                          npiece, hcoef, mask)
        else:
            VMath.mult_on_heads(dev, probs.ptr, K.ptr, Q.ptr, nbat, ntimes, nvec, nhead, npiece, hcoef)
            if mask:
                VMath.set_mh_attention_mask(dev, probs.ptr, nbat, ntimes, nhead, True)
            VMath.softmax_direct_on_axis(dev, probs.ptr, nbat * ntimes, ntimes, nhead)
            VMath.mix_values(dev, mixed.ptr, probs.ptr, V.ptr, nbat, ntimes, nvec, nhead, npiece)
        VMath.matmul(dev, y.ptr, Ow.ptr, mixed.ptr, nvec, n, nvec, False)
        VMath.add_bias(dev, y.ptr, y.ptr, Ob.ptr, n, nvec)
        y.saved = {"op": "mh_attention", "x": x, "key": key, "query": query, "value": value, "Kw": Kw, "Qw": Qw, "Vw": Vw,
                   "Ow": Ow, "K": K, "Q": Q, "V": V, "probs": probs, "mixed": mixed, "head_cnt": nhead,
                   "mask": mask, "coef": hcoef}
        return y

    # vtensor.cpp:3054-3195 (the math calls; gradient registration is the engine's business)
    def mh_attention_backprop(self, ygrad, fused=False):
        """Returns the 16 gradients by name (15 with ``fused=True``: one kai_attention_backward replaces the five or
        six calls between the projections, and the gradient of the probabilities is never formed).  ``g["x"]`` is the gradient of the tensor the operator was called on:
        zero, plus the gradient of each of key / query / value that IS that tensor (self-attention,
        vtensor.cpp:3168-3195).  The reference's set_zero there passes an element count where bytes are meant
        and clears a quarter of the buffer; the whole buffer is cleared here."""
        s = self.saved
        nbat, ntimes, nvec = self.shape
        nhead = s["head_cnt"]
        npiece = nvec // nhead
        dev = self.device
        n = nbat * ntimes
        T = lambda shape: Tensor(shape, dev)
        g = {name: T((nvec, nvec)) for name in ("Kw", "Qw", "Vw", "Ow")}
        g.update({name: T((nvec,)) for name in ("Kb", "Qb", "Vb", "Ob")})
        g.update({name: T(self.shape) for name in ("x", "key", "query", "value", "mixed", "K", "Q", "V")})
        g["probs"] = T((nbat, ntimes, ntimes, nhead))
        gy = ygrad.ptr
        VMath.add_bias_backward_b(dev, g["Ob"].ptr, gy, n, nvec, False)
        VMath.matmul_backward_w(dev, g["Ow"].ptr, gy, s["mixed"].ptr, nvec, n, nvec, False)
        VMath.matmul_backward_x(dev, g["mixed"].ptr, gy, s["Ow"].ptr, nvec, n, nvec, False)
        if fused:
            del g["probs"]
            VMath.attention_backward(dev, g["Q"].ptr, g["K"].ptr, g["V"].ptr, g["mixed"].ptr, s["probs"].ptr,
                                     s["mixed"].ptr, s["Q"].ptr, s["K"].ptr, s["V"].ptr, nbat, ntimes, nvec, nhead,
                                     npiece, s["coef"], s["mask"])
        else:
            VMath.mix_values_backward_prop(dev, g["probs"].ptr, g["mixed"].ptr, s["V"].ptr, nbat, ntimes, nvec, nhead,
                                           npiece)
            VMath.mix_values_backward_value(dev, g["V"].ptr, g["mixed"].ptr, s["probs"].ptr, nbat, ntimes, nvec, nhead,
                                            npiece)
            VMath.softmax_direct_on_axis_backward(dev, g["probs"].ptr, s["probs"].ptr, nbat, ntimes, nhead, s["coef"])
            if s["mask"]:
                VMath.set_mh_attention_mask(dev, g["probs"].ptr, nbat, ntimes, nhead, False)
            VMath.mult_on_heads_backward(dev, g["K"].ptr, g["probs"].ptr, s["Q"].ptr, nbat, ntimes, nvec, nhead, npiece)
            VMath.mult_on_heads_backward(dev, g["Q"].ptr, g["probs"].ptr, s["K"].ptr, nbat, ntimes, nvec, nhead, npiece)
        VMath.add_bias_backward_b(dev, g["Kb"].ptr, g["K"].ptr, n, nvec, False)
        VMath.add_bias_backward_b(dev, g["Qb"].ptr, g["Q"].ptr, n, nvec, False)
        VMath.add_bias_backward_b(dev, g["Vb"].ptr, g["V"].ptr, n, nvec, False)
        VMath.matmul_backward_w(dev, g["Kw"].ptr, g["K"].ptr, s["key"].ptr, nvec, n, nvec, False)
        VMath.matmul_backward_w(dev, g["Qw"].ptr, g["Q"].ptr, s["query"].ptr, nvec, n, nvec, False)
        VMath.matmul_backward_w(dev, g["Vw"].ptr, g["V"].ptr, s["value"].ptr, nvec, n, nvec, False)
        VMath.matmul_backward_x(dev, g["key"].ptr, g["K"].ptr, s["Kw"].ptr, nvec, n, nvec, False)
        VMath.matmul_backward_x(dev, g["query"].ptr, g["Q"].ptr, s["Qw"].ptr, nvec, n, nvec, False)
        VMath.matmul_backward_x(dev, g["value"].ptr, g["V"].ptr, s["Vw"].ptr, nvec, n, nvec, False)
        xsize = n * nvec
        VMath.set_zero(dev, g["x"].ptr, xsize * 4)
        for name in ("key", "query", "value"):
            if s[name] is s["x"]:
                VMath.add(dev, g["x"].ptr, g["x"].ptr, g[name].ptr, xsize)
        return g


def dense(x, w, b, actfunc="relu", leaky_alpha=None, fused=True, keep_pre=False):
    """The engine's ``dense`` layer formula activate(add(matmul(x, w), b)) (api/vconst.cpp:11).

    ``fused=False`` issues the three reference calls; ``fused=True`` the single-launch
    kai_dense_forward.  Returns (y, pre_activation or None)."""
    if not fused:
        pre = x.matmul(w).add(b)
        return pre.activate(actfunc, leaky_alpha), pre
    yvec, xvec = w.shape
    ndat = x.total_size() // xvec
    code = ACT[actfunc] if isinstance(actfunc, str) else int(actfunc)
    y = Tensor(x.shape[:-1] + (yvec,), x.device)
    pre = Tensor(y.shape, x.device) if keep_pre else None
    h = kai.hyper(leaky_alpha, x.device)
    VMath.dense_forward(x.device, y.ptr, pre.ptr if pre else None, w.ptr, b.ptr if b is not None else None, x.ptr,
                        yvec, ndat, xvec, code, h)
    return y, pre


# ---- recurrent layers: vtensor.cpp:2350-2522 (m_rnn) and 2524-2717 (m_rnn_backprop) ----------------------

VERR_SHAPE_RNN = 1307
_NGATES = {"rnn": 1, "lstm": 4, "gru": 3}


def rnn(x, wi, wr, bi, br, cell_type, rec_size, actfunc="tanh", leaky_alpha=None, forward=True, timesteps=None,
        use_state=False, batch_input_projection=False, fused_step=False):
    """One direction of a recurrent layer, as the engine's per-time-step loop issues it.

    ``x`` is ``[ntimes, ndat, ninp]`` (a sequence) or ``[ndat, ninp]`` (the same input at each of ``timesteps``
    steps); ``wi [ngates*nrec, ninp]``, ``wr [ngates*nrec, nrec]``, ``bi``/``br`` ``[ngates*nrec]`` or None.
    Per step: the recurrent gate product with acc = 0, the input gate product with acc = 1 (rnn and lstm keep
    both in one buffer), the bias adds, then the cell.  ``batch_input_projection=True`` is the additive fusion:
    the input products of all steps are issued as ONE call over ``ntimes*ndat`` rows before the loop and the
    recurrent product accumulates onto it, which gives the same sums (a + b == b + a).
    ``fused_step=True`` (lstm, gru; implies the batched input products for a sequence input) replaces the
    remaining calls of a step by ONE kai_lstm_step / kai_gru_step.
    Returns the ``[ndat, nrec]`` output and the tensors the backward pass needs."""
    if cell_type not in _NGATES:
        raise KaiError(8, "rnn cell type")
    ngates = _NGATES[cell_type]
    nrec = int(rec_size)
    in_seq = len(x.shape) == 3
    if len(wi.shape) != 2 or len(wr.shape) != 2:
        raise KaiError(VERR_SHAPE_RNN, "rnn")
    ntimes = x.shape[0] if in_seq else int(timesteps)
    ndat = x.shape[1] if in_seq else x.shape[0]
    ninp = x.shape[-1]
    if wi.shape != (ngates * nrec, ninp) or wr.shape != (ngates * nrec, nrec):
        raise KaiError(VERR_SHAPE_RNN, "rnn")
    use_bias = bi is not None
    if use_bias and (bi.shape != (ngates * nrec,) or br.shape != (ngates * nrec,)):
        raise KaiError(VERR_SHAPE_RNN, "rnn")
    dev = x.device
    code = ACT[actfunc] if isinstance(actfunc, str) else int(actfunc)
    halpha = kai.hyper(leaky_alpha, dev)
    recurs = Tensor((ntimes, ndat, nrec), dev)
    iaffines = Tensor((ntimes, ndat, ngates * nrec), dev)
    raffines = iaffines
    VMath.set_zero(dev, recurs.ptr, recurs.total_size() * 4)
    VMath.set_zero(dev, iaffines.ptr, iaffines.total_size() * 4)
    if cell_type == "gru":
        raffines = Tensor((ntimes, ndat, ngates * nrec), dev)
        VMath.set_zero(dev, raffines.ptr, raffines.total_size() * 4)
    states = None
    if cell_type == "lstm":
        states = Tensor((ntimes, ndat, nrec), dev)
        VMath.set_zero(dev, states.ptr, states.total_size() * 4)
    xsize, ysize = ndat * ninp, ndat * nrec
    asize = ngates * ysize
    f4 = 4
    fused_step = fused_step and cell_type in ("lstm", "gru")
    batched = (batch_input_projection or fused_step) and in_seq
    if batched:
        VMath.matmul(dev, iaffines.ptr, wi.ptr, x.ptr, ngates * nrec, ntimes * ndat, ninp, False)
    for n in range(ntimes):
        nt = n if forward else ntimes - n - 1
        pr = recurs.buf.offset(nt * ysize * f4)
        pai = iaffines.buf.offset(nt * asize * f4)
        par = raffines.buf.offset(nt * asize * f4)
        px = x.buf.offset(nt * xsize * f4) if in_seq else x.ptr
        if fused_step:
            pr_prev = recurs.buf.offset((nt - 1 if forward else nt + 1) * ysize * f4) if n > 0 else None
            if not batched:
                VMath.matmul(dev, pai, wi.ptr, px, ngates * nrec, ndat, ninp, True)
            pbi, pbr = (bi.ptr, br.ptr) if use_bias else (None, None)
            if cell_type == "lstm":
                ps = states.buf.offset(nt * ysize * f4)
                ps_prev = states.buf.offset((nt - 1 if forward else nt + 1) * ysize * f4) if n > 0 else None
                VMath.lstm_step(dev, pr, ps, ps_prev, pai, wr.ptr, pr_prev, pbi, pbr, ndat, nrec)
            else:
                ph_prev = recurs.buf.offset((nt - 1) * ysize * f4) if nt > 0 else None   # vmath.cu:4961
                VMath.gru_step(dev, pr, pai, par, wr.ptr, pr_prev, ph_prev, pbi, pbr, ndat, nrec)
            continue
        if n > 0:
            pr_prev = recurs.buf.offset((nt - 1 if forward else nt + 1) * ysize * f4)
            # with the input products already in place the recurrent one accumulates (rnn, lstm: same buffer)
            VMath.matmul(dev, par, wr.ptr, pr_prev, ngates * nrec, ndat, nrec, batched and raffines is iaffines)
        if not batched:
            VMath.matmul(dev, pai, wi.ptr, px, ngates * nrec, ndat, ninp, True)
        if use_bias:
            VMath.add_bias(dev, par, par, br.ptr, ndat, ngates * nrec)
            VMath.add_bias(dev, pai, pai, bi.ptr, ndat, ngates * nrec)
        if cell_type == "rnn":
            VMath.copy(dev, pr, pai, ysize)
            VMath.add(dev, pr, pr, pai, ysize)
            VMath.activate(dev, pr, pr, ndat, nrec, code, halpha)
        elif cell_type == "lstm":
            ps = states.buf.offset(nt * ysize * f4)
            ps_prev = states.buf.offset((nt - 1 if forward else nt + 1) * ysize * f4) if n > 0 else None
            VMath.lstm_process(dev, pr, ps, ps_prev, pai, ndat, nrec, ninp)
        else:
            VMath.gru_process(dev, pr, pai, par, nt, ntimes, ndat, nrec)
    y = Tensor((ndat, nrec), dev)
    src = states if (use_state and states is not None) else recurs
    VMath.copy(dev, y.ptr, src.buf.offset(((ntimes - 1) if forward else 0) * ysize * f4), ysize)
    saved = {"cell_type": cell_type, "forward": forward, "x": x, "wi": wi, "wr": wr, "use_bias": use_bias,
             "recurs": recurs, "iaffines": iaffines, "raffines": raffines, "states": states, "actfunc": code,
             "leaky_alpha": halpha, "ngates": ngates}
    return y, saved


def rnn_backprop(saved, ygrad, ytgrad, use_state=False):
    """vtensor.cpp:2524-2717.  ``ygrad [ndat, nrec]`` is used in place as the running gradient of the recurrent
    output (of the cell state for an lstm with ``use_state``), as there; ``ytgrad [ntimes, ndat, nrec]`` is the
    per-step gradient.  Returns {x, wi, wr[, bi, br]} gradients.  The lstm cell's gradient follows the
    reference's device kernel (vmath.cu:4899-4937)."""
    cell_type = saved["cell_type"]
    forward, ngates = saved["forward"], saved["ngates"]
    x, wi, wr = saved["x"], saved["wi"], saved["wr"]
    recurs, iaffines, raffines = saved["recurs"], saved["iaffines"], saved["raffines"]
    ntimes, ndat, nrec = ytgrad.shape
    ninp = x.shape[-1]
    in_seq = len(x.shape) == 3
    dev = x.device
    is_gru = cell_type == "gru"
    xgrad, wigrad, wrgrad = Tensor(x.shape, dev), Tensor(wi.shape, dev), Tensor(wr.shape, dev)
    aigrad = Tensor((ndat, ngates * nrec), dev)
    for t in (xgrad, wigrad, wrgrad):
        VMath.set_zero(dev, t.ptr, t.total_size() * 4)
    argrad = aigrad
    if is_gru:
        argrad = Tensor((ndat, ngates * nrec), dev)
        VMath.set_zero(dev, argrad.ptr, argrad.total_size() * 4)
    out = {"x": xgrad, "wi": wigrad, "wr": wrgrad}
    if saved["use_bias"]:
        out["bi"], out["br"] = Tensor((ngates * nrec,), dev), Tensor((ngates * nrec,), dev)
        VMath.set_zero(dev, out["bi"].ptr, ngates * nrec * 4)
        VMath.set_zero(dev, out["br"].ptr, ngates * nrec * 4)
    pgr = ygrad.ptr
    pgs = None
    states = saved["states"]
    use_state = use_state and cell_type == "lstm"
    if cell_type == "lstm":
        # vtensor.cpp:2614-2631: with use_state the incoming gradient is that of the state and the output's
        # gradient starts at zero, otherwise the other way round
        fresh = Tensor(ygrad.shape, dev)
        VMath.set_zero(dev, fresh.ptr, fresh.total_size() * 4)
        if use_state:
            pgs, pgr = ygrad.ptr, fresh.ptr
        else:
            pgs = fresh.ptr
    xsize, ysize = ndat * ninp, ndat * nrec
    asize = ngates * ysize
    f4 = 4
    for n in range(ntimes):
        nt = ntimes - n - 1 if forward else n
        pr = recurs.buf.offset(nt * ysize * f4)
        pai = iaffines.buf.offset(nt * asize * f4)
        par = raffines.buf.offset(nt * asize * f4)
        px = x.buf.offset(nt * xsize * f4) if in_seq else x.ptr
        pgx = xgrad.buf.offset(nt * xsize * f4) if in_seq else xgrad.ptr
        pg_step = pgs if use_state else pgr
        VMath.add(dev, pg_step, pg_step, ytgrad.buf.offset(nt * ysize * f4), ysize)
        if cell_type == "rnn":
            VMath.activate_backward_with_y(dev, aigrad.ptr, pgr, pr, ndat, nrec, saved["actfunc"], saved["leaky_alpha"])
        elif cell_type == "lstm":
            ps_prev = states.buf.offset((nt - 1 if forward else nt + 1) * ysize * f4) if n < ntimes - 1 else None
            VMath.lstm_process_backward(dev, pgr, pgs, aigrad.ptr, ps_prev, pai, ndat, nrec, ninp)
        else:
            VMath.gru_process_backward(dev, pgr, aigrad.ptr, argrad.ptr, pr, pai, par, nt, ntimes, ndat, nrec)
        if saved["use_bias"]:
            VMath.add_bias_backward_b(dev, out["bi"].ptr, aigrad.ptr, ndat, ngates * nrec, True)
            VMath.add_bias_backward_b(dev, out["br"].ptr, argrad.ptr, ndat, ngates * nrec, True)
        VMath.matmul_backward_w(dev, wigrad.ptr, aigrad.ptr, px, ngates * nrec, ndat, ninp, True)
        if n < ntimes - 1:
            pr_prev = recurs.buf.offset((nt - 1 if forward else nt + 1) * ysize * f4)
            VMath.matmul_backward_w(dev, wrgrad.ptr, argrad.ptr, pr_prev, ngates * nrec, ndat, nrec, True)
        VMath.matmul_backward_x(dev, pgx, aigrad.ptr, wi.ptr, ngates * nrec, ndat, ninp, False)
        VMath.matmul_backward_x(dev, pgr, argrad.ptr, wr.ptr, ngates * nrec, ndat, nrec, is_gru)
    return out
