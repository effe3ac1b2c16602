"""Tensor-level graphs of the benchmark configurations, built through the REAL
reference frontend (tests/refpoly.py).  Test infrastructure only.

gpt2_forward follows the topology of the reference's GPT-2 builder
(src/modelzoo/models/gpt2.c:320-526: one-hot embedding, pre-LayerNorm blocks,
Conv1D-style linears, additive causal mask, softmax, GELU, tied LM head, a
realize barrier after every op) and adds the bf16 variant the benchmark names:
bf16 buffers, CAST to f32 in front of every reduction (matmul, LayerNorm
statistics, softmax max/sum, embedding sum) and CAST back to bf16 after it.
"""
import math

import numpy as np

import refpoly as R


class GPT2Config:
    def __init__(self, n_layer=12, n_head=12, d_model=768, vocab=50257, ctx=1024, batch=8, eps=1e-5):
        self.n_layer, self.n_head, self.d_model, self.vocab, self.ctx, self.batch, self.eps = \
            n_layer, n_head, d_model, vocab, ctx, batch, eps

    def key(self):
        return f"L{self.n_layer}_H{self.n_head}_D{self.d_model}_V{self.vocab}_T{self.ctx}_B{self.batch}"


GPT2_SMALL = GPT2Config()
GPT2_TINY = GPT2Config(n_layer=2, n_head=2, d_model=32, vocab=97, ctx=16, batch=2)


def _embedding(c, table, n_rows, d, idx, idx_shape, arange, wdt):
    """out[..., j] = sum_v where(idx[...] == arange[v], table[v, j], 0)  (src/modelzoo/models/gpt2.c:93-153)."""
    nd = len(idx_shape)
    idx_e = idx.reshape(idx_shape + (1,)).expand(idx_shape + (n_rows,))
    ar_e = arange.reshape((1,) * nd + (n_rows,)).expand(idx_shape + (n_rows,))
    mask = idx_e.eq(ar_e).reshape(idx_shape + (n_rows, 1)).expand(idx_shape + (n_rows, d))
    tbl = table.reshape((1,) * nd + (n_rows, d)).expand(idx_shape + (n_rows, d))
    if wdt != R.F32:
        tbl = tbl.cast(R.F32)
    sel = mask.where(tbl, c.const(0.0))
    out = sel.reduce_axes("ADD", [nd]).reshape(idx_shape + (d,))
    return out.cast(wdt) if wdt != R.F32 else out


def _linear(x, w, b, wdt):
    """x @ w + b with HF Conv1D weight layout (in, out); f32 accumulate."""
    if wdt != R.F32:
        y = x.cast(R.F32).dot(w.cast(R.F32)).cast(wdt)
    else:
        y = x.dot(w)
    if b is not None:
        y = y + b.reshape((1,) * (len(y.shape) - 1) + (b.shape[-1],)).expand(y.shape)
    return y


def _layernorm(x, w, b, eps, wdt):
    d = x.shape[-1]
    xf = x.cast(R.F32) if wdt != R.F32 else x
    y = xf.layernorm(eps)
    if wdt != R.F32:
        y = y.cast(wdt)
    bc = (1,) * (len(x.shape) - 1) + (d,)
    return y * w.reshape(bc).expand(x.shape) + b.reshape(bc).expand(x.shape)


def gpt2_forward(c, cfg, wdt=R.BF16, hidden_only=False):
    """Returns (sink, bufs) where bufs maps names to buffer T's; logits go to bufs['output'].
    With hidden_only the graph ends after the last block: the residual stream [B, T, D] goes
    to bufs['hidden'] and the final LayerNorm and the vocabulary projection are left out."""
    V, D, H, L, T, B = cfg.vocab, cfg.d_model, cfg.n_head, cfg.n_layer, cfg.ctx, cfg.batch
    hd = D // H
    bufs = {}

    def P(name, shape, dt=None):
        bufs[name] = c.buffer(shape, wdt if dt is None else dt, name=name)
        return bufs[name]

    wte = P("wte.weight", (V, D))
    wpe = P("wpe.weight", (T, D))
    layers = []
    for i in range(L):
        p = f"h.{i}."
        layers.append(dict(
            ln1_w=P(p + "ln_1.weight", (D,)), ln1_b=P(p + "ln_1.bias", (D,)),
            attn_w=P(p + "attn.c_attn.weight", (D, 3 * D)), attn_b=P(p + "attn.c_attn.bias", (3 * D,)),
            proj_w=P(p + "attn.c_proj.weight", (D, D)), proj_b=P(p + "attn.c_proj.bias", (D,)),
            ln2_w=P(p + "ln_2.weight", (D,)), ln2_b=P(p + "ln_2.bias", (D,)),
            fc_w=P(p + "mlp.c_fc.weight", (D, 4 * D)), fc_b=P(p + "mlp.c_fc.bias", (4 * D,)),
            fc2_w=P(p + "mlp.c_proj.weight", (4 * D, D)), fc2_b=P(p + "mlp.c_proj.bias", (D,))))
    lnf_w, lnf_b = P("ln_f.weight", (D,)), P("ln_f.bias", (D,))
    # token ids, positions and the aranges are FLOAT buffers, as in the reference
    x = P("x", (B, T), R.F32)
    out = P("output", (B, T, V))
    pos = P("positions", (1, T), R.F32)
    arange = P("arange", (T,), R.F32)
    varange = P("vocab_arange", (V,), R.F32)

    tok = _embedding(c, wte, V, D, x, (B, T), varange, wdt).contiguous()
    pe = _embedding(c, wpe, T, D, pos, (1, T), arange, wdt).contiguous()
    h = (tok + pe.expand((B, T, D))).contiguous()

    row = arange.reshape((T, 1)).expand((T, T))
    col = arange.reshape((1, T)).expand((T, T))
    mask = row.lt(col).where(c.const(-1e9, wdt), c.const(0.0, wdt)).reshape((1, 1, T, T)).contiguous()

    scale = 1.0 / math.sqrt(hd)
    for lp in layers:
        ln1 = _layernorm(h, lp["ln1_w"], lp["ln1_b"], cfg.eps, wdt).contiguous()
        qkv = _linear(ln1, lp["attn_w"], lp["attn_b"], wdt).contiguous()
        q = qkv.shrink(((0, B), (0, T), (0, D))).contiguous()
        k = qkv.shrink(((0, B), (0, T), (D, 2 * D))).contiguous()
        v = qkv.shrink(((0, B), (0, T), (2 * D, 3 * D))).contiguous()
        q = q.reshape((B, T, H, hd)).permute((0, 2, 1, 3))
        k = k.reshape((B, T, H, hd)).permute((0, 2, 1, 3))
        v = v.reshape((B, T, H, hd)).permute((0, 2, 1, 3))
        kt = k.permute((0, 1, 3, 2))
        if wdt != R.F32:
            scores = q.cast(R.F32).dot(kt.cast(R.F32)).cast(wdt).contiguous()
        else:
            scores = q.dot(kt).contiguous()
        scores = (scores * c.const(scale, wdt) + mask.expand((B, H, T, T))).contiguous()
        if wdt != R.F32:
            attn = scores.cast(R.F32).softmax(-1).cast(wdt).contiguous()
            ctxv = attn.cast(R.F32).dot(v.cast(R.F32)).cast(wdt).contiguous()
        else:
            attn = scores.softmax(-1).contiguous()
            ctxv = attn.dot(v).contiguous()
        merged = ctxv.permute((0, 2, 1, 3)).reshape((B, T, D))
        a_out = _linear(merged, lp["proj_w"], lp["proj_b"], wdt).contiguous()
        h = (h + a_out).contiguous()
        ln2 = _layernorm(h, lp["ln2_w"], lp["ln2_b"], cfg.eps, wdt).contiguous()
        ff = _linear(ln2, lp["fc_w"], lp["fc_b"], wdt).contiguous()
        ff = ff.gelu().contiguous()
        ff = _linear(ff, lp["fc2_w"], lp["fc2_b"], wdt).contiguous()
        h = (h + ff).contiguous()

    if hidden_only:
        hidden = P("hidden", (B, T, D))
        return c.sink((hidden, h)), bufs
    h = _layernorm(h, lnf_w, lnf_b, cfg.eps, wdt).contiguous()
    wte_t = wte.reshape((V, D)).permute((1, 0))
    if wdt != R.F32:
        logits = h.cast(R.F32).dot(wte_t.cast(R.F32)).cast(wdt)
    else:
        logits = h.dot(wte_t)
    sink = c.sink((out, logits))
    return sink, bufs


def gpt2_inputs(cfg, bufs, seed=3, wdt=R.BF16):
    """Random-init weights and inputs per the benchmark config: weights ~ N(0, 0.02),
    LayerNorm weights 1, biases 0, token ids uniform in [0, vocab) stored as floats."""
    g = np.random.default_rng(seed)
    arrays = {}
    for name, t in bufs.items():
        n = int(np.prod(t.shape))
        if name == "x":
            a = g.integers(0, cfg.vocab, n).astype(np.float32)
        elif name in ("positions", "arange"):
            a = np.arange(cfg.ctx, dtype=np.float32)
        elif name == "vocab_arange":
            a = np.arange(cfg.vocab, dtype=np.float32)
        elif name == "output":
            a = np.zeros(n, np.float32)
        elif name.endswith("ln_1.weight") or name.endswith("ln_2.weight") or name == "ln_f.weight":
            a = np.ones(n, np.float32)
        elif name.endswith(".bias"):
            a = np.zeros(n, np.float32)
        else:
            a = g.normal(0.0, 0.02, n).astype(np.float32)
        if t.dt == R.BF16:
            a = R.f32_to_bf16_bits(a)
        elif t.dt == R.F16:
            a = a.astype(np.float16)
        arrays[t] = a
    return arrays


def fused_rowops(c, rows, cols):
    """Config 2: y = clamp(exp2(a*b + c), -4, 4); sum, max, softmax, LayerNorm over the last axis."""
    a, b, d = (c.buffer((rows, cols), name=n) for n in ("a", "b", "c"))
    y = (a * b + d).exp2().clamp(-4, 4)
    outs = {"sum": c.buffer((rows,), name="sum"), "max": c.buffer((rows,), name="max"),
            "softmax": c.buffer((rows, cols), name="softmax"), "layernorm": c.buffer((rows, cols), name="layernorm")}
    sinks = {"sum": c.sink((outs["sum"], y.sum())), "max": c.sink((outs["max"], y.max())),
             "softmax": c.sink((outs["softmax"], y.softmax())),
             "layernorm": c.sink((outs["layernorm"], y.layernorm(1e-5)))}
    return (a, b, d), outs, sinks


def matmul_bf16(c, m, n, k, transposed_b=False, batch=None, transposed_a=False):
    """Config 3: C = A@B, bf16 inputs, f32 accumulate and output.  transposed_a / transposed_b:
    the operand is stored (k, m) / (n, k) and permuted in the graph (the forms the backward
    pass of a linear layer produces: dX = dY W^T, dW = X^T dY)."""
    if transposed_a:
        assert batch is None
        At = c.buffer((k, m), R.BF16, name="A")
        Bm = c.buffer((n, k), R.BF16, name="B") if transposed_b else c.buffer((k, n), R.BF16, name="B")
        b = Bm.permute((1, 0)) if transposed_b else Bm
        O = c.buffer((m, n), R.F32, name="C")
        return At, Bm, O, c.sink((O, At.permute((1, 0)).cast(R.F32).dot(b.cast(R.F32))))
    a_shape = (m, k) if batch is None else (batch, m, k)
    A = c.buffer(a_shape, R.BF16, name="A")
    if transposed_b:
        Bm = c.buffer((n, k), R.BF16, name="B")
        b = Bm.permute((1, 0))
    else:
        Bm = c.buffer((k, n), R.BF16, name="B")
        b = Bm
    O = c.buffer(a_shape[:-1] + (n,), R.F32, name="C")
    sink = c.sink((O, A.cast(R.F32).dot(b.cast(R.F32))))
    return A, Bm, O, sink


def matmul_bf16_over_two_ranges(c, b, t, m, n, time_major_a=False):
    """C[m, n] = sum over (b, t) of X[b, t, m] * Y[b, t, n]: the weight gradient of a linear
    layer over a batch of sequences, as one REDUCE over two ranges.  time_major_a: X is
    stored [t, b, m] and permuted in the graph, so its two reduce strides do not nest in
    the order Y's do."""
    X = c.buffer((t, b, m) if time_major_a else (b, t, m), R.BF16, name="A")
    Y = c.buffer((b, t, n), R.BF16, name="B")
    O = c.buffer((m, n), R.F32, name="C")
    x = X.permute((1, 0, 2)) if time_major_a else X
    p = x.cast(R.F32).reshape((b, t, m, 1)).expand((b, t, m, n)) * Y.cast(R.F32).reshape((b, t, 1, n)).expand((b, t, m, n))
    return X, Y, O, c.sink((O, p.reduce_axes("ADD", (0, 1)).reshape((m, n))))


def attention_bf16(c, batch=8, heads=12, ctx=1024, hd=64, mask_buffer=False, dt=None):
    """The attention block of gpt2_forward on its own: q, k, v as [B, T, H*hd] bf16 buffers
    (heads interleaved along the feature axis, as the qkv projection leaves them), additive
    causal mask built from an arange buffer (or, with mask_buffer, any additive [T, T] bf16
    mask handed in as a buffer), softmax in fp32, heads merged back into [B, T, H*hd] by a
    separate copy kernel (in gpt2_forward the projection matmul reads the per-head layout
    instead)."""
    D = heads * hd
    dt = R.BF16 if dt is None else dt   # the 16-bit type of q, k, v, scores and output
    q, k, v = (c.buffer((batch, ctx, D), dt, name=n) for n in ("q", "k", "v"))
    out = c.buffer((batch, ctx, D), dt, name="out")
    bufs = dict(q=q, k=k, v=v, out=out)
    if mask_buffer:
        bufs["mask"] = c.buffer((ctx, ctx), dt, name="mask")
        mask = bufs["mask"].reshape((1, 1, ctx, ctx))
    else:
        bufs["arange"] = arange = c.buffer((ctx,), R.F32, name="arange")
        row = arange.reshape((ctx, 1)).expand((ctx, ctx))
        col = arange.reshape((1, ctx)).expand((ctx, ctx))
        mask = row.lt(col).where(c.const(-1e9, dt), c.const(0.0, dt)).reshape((1, 1, ctx, ctx)).contiguous()
    qh = q.reshape((batch, ctx, heads, hd)).permute((0, 2, 1, 3))
    kh = k.reshape((batch, ctx, heads, hd)).permute((0, 2, 1, 3))
    vh = v.reshape((batch, ctx, heads, hd)).permute((0, 2, 1, 3))
    scores = qh.cast(R.F32).dot(kh.permute((0, 1, 3, 2)).cast(R.F32)).cast(dt).contiguous()
    scores = (scores * c.const(1.0 / math.sqrt(hd), dt) + mask.expand((batch, heads, ctx, ctx))).contiguous()
    attn = scores.cast(R.F32).softmax(-1).cast(dt).contiguous()
    ctxv = attn.cast(R.F32).dot(vh.cast(R.F32)).cast(dt).contiguous()
    merged = ctxv.permute((0, 2, 1, 3)).reshape((batch, ctx, D))
    return bufs, c.sink((out, merged))


def mlp_train_step(c, batch=4096, d_in=784, d_hid=512, d_out=10, lr=0.01):
    """Config 1: 2-layer MLP (weights stored (out, in) as the reference's model_mlp.c does),
    softmax cross-entropy against one-hot labels, reverse-mode gradients from the
    reference's poly_grad, one SGD step.  Returns (bufs, sink): the sink stores logits and
    loss and updates the four parameters in place (ASSIGN)."""
    X = c.buffer((batch, d_in), name="X")
    W1 = c.buffer((d_hid, d_in), name="W1")
    b1 = c.buffer((d_hid,), name="b1")
    W2 = c.buffer((d_out, d_hid), name="W2")
    b2 = c.buffer((d_out,), name="b2")
    Y = c.buffer((batch, d_out), name="Y")  # one-hot labels
    logits_out = c.buffer((batch, d_out), name="logits")
    loss_out = c.buffer((1,), name="loss")
    h = (X.dot(W1.permute((1, 0))) + b1.reshape((1, d_hid)).expand((batch, d_hid))).relu()
    logits = h.dot(W2.permute((1, 0))) + b2.reshape((1, d_out)).expand((batch, d_out))
    logp = logits.log_softmax(-1)
    loss = (logp * Y).sum().sum(0) * c.const(-1.0 / batch)
    pairs = []
    for p in (W1, b1, W2, b2):
        n = int(np.prod(p.shape))
        g = T_grad(c, loss, p, n)
        pairs.append((p, p.reshape((n,)) - g * c.const(lr)))
    bufs = dict(X=X, W1=W1, b1=b1, W2=W2, b2=b2, Y=Y, logits=logits_out, loss=loss_out)
    return bufs, c.sink_mixed([(logits_out, logits), (loss_out, loss.reshape((1,)))], pairs)


def T_grad(c, loss, param, numel):
    """d loss / d param as a flat tensor (reference poly_grad, src/autograd.c:773)."""
    u = c.L.poly_grad(c.ctx, loss.u, param.buf)
    if not u:
        raise RuntimeError("poly_grad failed")
    return R.T(c, u, (numel,), param.dt)


def adamw_step(c, numel, lr=3e-4, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.1):
    """One AdamW update of a flat parameter, built the way the reference's training graph
    builds it (src/instance.c:1162-1224): decoupled decay, moments, bias corrections read
    from one-element buffers and expanded, three in-place ASSIGNs (param, m, v)."""
    p, g, m, v = (c.buffer((numel,), name=n) for n in ("p", "g", "m", "v"))
    bc1, bc2 = c.buffer((1,), name="bc1"), c.buffer((1,), name="bc2")
    p_cur = p * c.const(1.0 - lr * weight_decay)
    m_new = c.const(beta1) * m + c.const(1.0 - beta1) * g
    v_new = c.const(beta2) * v + c.const(1.0 - beta2) * (g * g)
    m_hat = m_new * bc1.expand((numel,))
    v_hat = v_new * bc2.expand((numel,))
    denom = v_hat.sqrt() + c.const(eps)
    p_new = p_cur - c.const(lr) * (m_hat * denom.un("RECIPROCAL"))
    bufs = dict(p=p, g=g, m=m, v=v, bc1=bc1, bc2=bc2)
    return bufs, c.sink_assign((p, p_new), (m, m_new), (v, v_new))


BLOCK_PARAMS = ("ln1_w", "ln1_b", "attn_w", "attn_b", "proj_w", "proj_b", "ln2_w", "ln2_b", "fc_w", "fc_b", "fc2_w", "fc2_b",
                "lnf_w", "lnf_b", "head_w")


LAYER_PARAMS = BLOCK_PARAMS[:12]


def train_param_names(n_blocks):
    """Parameter names of gpt2_block_train_step: one block keeps the bare names, several
    blocks prefix theirs with h<i>. (the final LayerNorm and the head stay bare)."""
    if n_blocks == 1:
        return list(BLOCK_PARAMS)
    return [f"h{i}.{n}" for i in range(n_blocks) for n in LAYER_PARAMS] + ["lnf_w", "lnf_b", "head_w"]


def gpt2_block_train_step(c, batch=4, ctx=1024, d_model=1024, heads=16, vocab=50257, lr=3e-4, beta1=0.9, beta2=0.999,
                          eps=1e-8, weight_decay=0.1, ln_eps=1e-5, head_vd=True, n_blocks=1):
    """n_blocks transformer blocks of config 5 (GPT-2 medium shapes; 24 of them are the
    whole model above the embedding) with the final LayerNorm, the vocabulary projection and
    next-token cross-entropy, reverse-mode gradients from the reference's poly_grad
    (src/autograd.c:773) and an AdamW update of every parameter (src/instance.c:1162-1224).
    Mixed precision: fp32 master parameters and optimizer state, bf16 copies of the weights
    and bf16 activations for the matmuls, fp32 reductions.  The first block's input
    activations stand in for the embedding below it.
    Returns (bufs, sink): the sink stores the loss and updates p, m, v of every parameter."""
    B, T, D, H, V = batch, ctx, d_model, heads, vocab
    hd = D // H
    shapes = dict(ln1_w=(D,), ln1_b=(D,), attn_w=(D, 3 * D), attn_b=(3 * D,), proj_w=(D, D), proj_b=(D,), ln2_w=(D,),
                  ln2_b=(D,), fc_w=(D, 4 * D), fc_b=(4 * D,), fc2_w=(4 * D, D), fc2_b=(D,), lnf_w=(D,), lnf_b=(D,),
                  head_w=(V, D) if head_vd else (D, V))      # (V, D): tied-embedding layout, as GPT-2 stores it
    names = train_param_names(n_blocks)
    bufs = {}
    P = {}
    for name in names:
        shape = shapes[name.split(".")[-1]]
        P[name] = bufs[name] = c.buffer(shape, R.F32, name=name)
        bufs[name + ".m"] = c.buffer(shape, R.F32, name=name + ".m")
        bufs[name + ".v"] = c.buffer(shape, R.F32, name=name + ".v")
    h0 = bufs["h0"] = c.buffer((B, T, D), R.BF16, name="h0")
    target = bufs["target"] = c.buffer((B * T,), R.F32, name="target")     # class ids as floats (sparse cross-entropy)
    arange = bufs["arange"] = c.buffer((T,), R.F32, name="arange")
    bc1, bc2 = c.buffer((1,), name="bc1"), c.buffer((1,), name="bc2")
    bufs["bc1"], bufs["bc2"] = bc1, bc2
    loss_out = bufs["loss"] = c.buffer((1,), R.F32, name="loss")
    W = {k: v.cast(R.BF16).contiguous() for k, v in P.items()}             # bf16 working copies, one cast kernel each

    row = arange.reshape((T, 1)).expand((T, T))
    col = arange.reshape((1, T)).expand((T, T))
    mask = row.lt(col).where(c.const(-1e9, R.BF16), c.const(0.0, R.BF16)).reshape((1, 1, T, T)).contiguous()
    wdt = R.BF16
    h = h0
    for i in range(n_blocks):
        w = (lambda n: W[n]) if n_blocks == 1 else (lambda n, i=i: W[f"h{i}.{n}"])
        ln1 = _layernorm(h, w("ln1_w"), w("ln1_b"), ln_eps, wdt).contiguous()
        qkv = _linear(ln1, w("attn_w"), w("attn_b"), wdt).contiguous()
        q = qkv.shrink(((0, B), (0, T), (0, D))).contiguous().reshape((B, T, H, hd)).permute((0, 2, 1, 3))
        k = qkv.shrink(((0, B), (0, T), (D, 2 * D))).contiguous().reshape((B, T, H, hd)).permute((0, 2, 1, 3))
        v = qkv.shrink(((0, B), (0, T), (2 * D, 3 * D))).contiguous().reshape((B, T, H, hd)).permute((0, 2, 1, 3))
        scores = q.cast(R.F32).dot(k.permute((0, 1, 3, 2)).cast(R.F32)).cast(wdt).contiguous()
        scores = (scores * c.const(1.0 / math.sqrt(hd), wdt) + mask.expand((B, H, T, T))).contiguous()
        attn = scores.cast(R.F32).softmax(-1).cast(wdt).contiguous()
        ctxv = attn.cast(R.F32).dot(v.cast(R.F32)).cast(wdt).contiguous()
        merged = ctxv.permute((0, 2, 1, 3)).reshape((B, T, D))
        h1 = (h + _linear(merged, w("proj_w"), w("proj_b"), wdt).contiguous()).contiguous()
        ln2 = _layernorm(h1, w("ln2_w"), w("ln2_b"), ln_eps, wdt).contiguous()
        ff = _linear(ln2, w("fc_w"), w("fc_b"), wdt).contiguous().gelu().contiguous()
        h = (h1 + _linear(ff, w("fc2_w"), w("fc2_b"), wdt).contiguous()).contiguous()
    lnf = _layernorm(h, W["lnf_w"], W["lnf_b"], ln_eps, wdt).contiguous()
    hw = W["head_w"].permute((1, 0)) if head_vd else W["head_w"]
    logits = lnf.reshape((B * T, D)).cast(R.F32).dot(hw.cast(R.F32)).contiguous()   # fp32 logits
    loss = logits.cross_entropy(target)
    assigns = []
    grads = {}
    if n_blocks > 1:
        # one reverse pass for all parameters, as the reference's own training graph takes
        # them (poly_grad_many, src/instance.c:876-963); a pass per parameter grows with the
        # square of the depth
        import ctypes as C
        wrts = (C.c_void_p * len(names))(*[P[nm].buf for nm in names])
        outs = (C.c_void_p * len(names))()
        if c.L.poly_grad_many(c.ctx, loss.u, None, wrts, len(names), outs) != 0:
            raise RuntimeError("poly_grad_many failed")
        for nm, u in zip(names, outs):
            grads[nm] = R.T(c, u, P[nm].shape, P[nm].dt).reshape((int(np.prod(P[nm].shape)),))
    for name in names:
        p, m, vv = P[name], bufs[name + ".m"], bufs[name + ".v"]
        n = int(np.prod(p.shape))
        g = grads[name] if name in grads else T_grad(c, loss, p, n)
        pf, mf, vf = p.reshape((n,)), m.reshape((n,)), vv.reshape((n,))
        m_new = c.const(beta1) * mf + c.const(1.0 - beta1) * g
        v_new = c.const(beta2) * vf + c.const(1.0 - beta2) * (g * g)
        denom = (v_new * bc2.expand((n,))).sqrt() + c.const(eps)
        p_new = pf * c.const(1.0 - lr * weight_decay) - c.const(lr) * ((m_new * bc1.expand((n,))) * denom.un("RECIPROCAL"))
        assigns += [(p, p_new), (m, m_new), (vv, v_new)]
    return bufs, c.sink_mixed([(loss_out, loss.reshape((1,)))], assigns)


def gpt2_block_train_inputs(bufs, batch, ctx, vocab, seed=4):
    """Seeded inputs for gpt2_block_train_step: weights ~ N(0, 0.02), LayerNorm weights 1,
    biases 0, optimizer state 0, activations ~ N(0, 1) as bf16, uniform random targets."""
    g = np.random.default_rng(seed)
    arrays = {}
    for name, t in bufs.items():
        n = int(np.prod(t.shape))
        if name == "h0":
            a = R.f32_to_bf16_bits(g.normal(0.0, 1.0, n).astype(np.float32))
        elif name == "target":
            a = g.integers(0, vocab, n).astype(np.float32)
        elif name == "arange":
            a = np.arange(ctx, dtype=np.float32)
        elif name == "bc1":
            a = np.array([1.0 / (1.0 - 0.9)], np.float32)
        elif name == "bc2":
            a = np.array([1.0 / (1.0 - 0.999)], np.float32)
        elif name.endswith(".m") or name.endswith(".v") or name == "loss" or name.endswith("_b"):
            a = np.zeros(n, np.float32)
        elif name.split(".")[-1] in ("ln1_w", "ln2_w", "lnf_w"):
            a = np.ones(n, np.float32)
        else:
            a = g.normal(0.0, 0.02, n).astype(np.float32)
        arrays[t] = a
    return arrays
