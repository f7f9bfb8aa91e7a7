"""Plain float64 numpy statement of the Vetipel design, one function per mechanism.  Test infrastructure only: slow, whole
sequences, no cache, no batching - the product (the stack engine) never touches it and shares no code with it.

Vetipel is a pre-norm decoder stack, x <- x + mixer(n1(x)), x <- x + ff(n2(x)), whose residual is kept in `streams` copies joined by
hyper-connections, whose norms carry their weight as an offset from one, and whose mixers are three kinds of attention:
  'attention'         grouped-query, no rotation, a linear distance penalty per head, a sliding window, sigmoid weights (no
                      normalisation over keys) with a per-head offset, and a per-head sigmoid output gate;
  'latent_attention'  keys and values expanded from one low-rank latent per token, plus one rotated key part shared by the heads;
                      causal softmax;
  'attention_2'       grouped-query with projection biases, unit-RMS queries and keys, a per-head temperature, a logarithmic
                      distance penalty, a chunked mask, a softmax whose denominator holds a per-head sink, and the output gate.
The feed-forward is W_down relu(W_up h)^2.

Notation: n tokens, width W; H query heads, G key/value heads, D query/key size, E value size.  `w` is a dict name -> float64
array with the checkpoint's names; `cfg` is the parsed config.json."""
import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def offset_rms_norm(x, weight, eps, offset=1.0):
    """x / sqrt(mean(x^2) + eps) * (offset + weight) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * (offset + weight)


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rotate_pairs(x, positions, dims, base):
    """x [n, ..., D]: dimensions (2i, 2i + 1), i < dims / 2, turn by positions * base^(-2i / dims); the rest pass."""
    if not dims:
        return x
    freq = base ** (-2.0 * np.arange(dims // 2, dtype=np.float64) / dims)
    ang = positions.astype(np.float64)[:, None] * freq[None, :]
    shape = (x.shape[0], ) + (1, ) * (x.ndim - 2) + (dims // 2, )
    c, s = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    even, odd = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.copy()
    out[..., 0:dims:2] = even * c - odd * s
    out[..., 1:dims:2] = odd * c + even * s
    return out


def visible(n, kind, size):
    """bool [n, n]: may row i look at column j."""
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    vis = j <= i
    if kind == 'window':
        vis &= (i - j) < size
    elif kind == 'chunk':
        vis &= (i // size) == (j // size)
    return vis


def distance(n):
    return (np.arange(n)[:, None] - np.arange(n)[None, :]).astype(np.float64)


def head_gate(h, w_g):
    """[n, H]: one sigmoid gate per head from the mixer's input."""
    return sigmoid(h @ w_g.T)


def sigmoid_window_attention(h, w, p, m):
    """Mixer 'attention'.  h [n, W] -> [n, W]."""
    n = h.shape[0]
    H, G, D, E = m['heads'], m['kv_heads'], m['dim'], m['vdim']
    q = (h @ w[p + 'q'].T).reshape(n, H, D)
    k = (h @ w[p + 'k'].T).reshape(n, G, D)
    v = (h @ w[p + 'v'].T).reshape(n, G, E)
    vis, dist = visible(n, 'window', m['mask']['size']), distance(n)
    gate = head_gate(h, w[p + 'g'])
    out = np.zeros((n, H, E))
    for a in range(H):
        g = a // (H // G)
        slope = 2.0 ** (-8.0 * (a + 1) / H)
        s = (q[:, a] @ k[:, g].T) * m['scale'] - slope * dist
        wt = np.where(vis, sigmoid(s + w[p + 'pb'][a]), 0.0)
        out[:, a] = (wt @ v[:, g]) * gate[:, a:a + 1]
    return out.reshape(n, H * E) @ w[p + 'o'].T


def latent_attention(h, w, p, m, eps):
    """Mixer 'latent_attention'.  Per token one latent c (RMS-normed, plain weight) and one rotated key part; per head the
    unrotated key and the value are linear in c."""
    n = h.shape[0]
    H, D, R, E, C = m['heads'], m['dim'], m['rot_dim'], m['vdim'], m['kv_rank']
    pos = np.arange(n)
    q = (h @ w[p + 'q'].T).reshape(n, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_pairs(q[..., D:], pos, m['rot']['dims'], m['rot']['base'])
    down = h @ w[p + 'dkv'].T
    c = offset_rms_norm(down[:, :C], w[p + 'dkv.norm'], eps, offset=0.0)
    k_rot = rotate_pairs(down[:, C:], pos, m['rot']['dims'], m['rot']['base'])       # [n, R], shared by the heads
    k_plain = (c @ w[p + 'uk'].T).reshape(n, H, D)
    v = (c @ w[p + 'uv'].T).reshape(n, H, E)
    vis = visible(n, 'causal', 0)
    out = np.zeros((n, H, E))
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m['scale']
        s = np.where(vis, s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, a] = (e / e.sum(axis=1, keepdims=True)) @ v[:, a]
    return out.reshape(n, H * E) @ w[p + 'o'].T


def sink_chunk_attention(h, w, p, m, eps):
    """Mixer 'attention_2'.  Softmax over the visible keys of the row's chunk and one sink logit that has no value."""
    n = h.shape[0]
    H, G, D, E = m['heads'], m['kv_heads'], m['dim'], m['vdim']
    q = unit_rms((h @ w[p + 'q'].T + w[p + 'q.b']).reshape(n, H, D), eps)
    k = unit_rms((h @ w[p + 'k'].T + w[p + 'k.b']).reshape(n, G, D), eps)
    v = (h @ w[p + 'v'].T + w[p + 'v.b']).reshape(n, G, E)
    vis, dist = visible(n, 'chunk', m['mask']['size']), distance(n)
    gate = head_gate(h, w[p + 'g'])
    out = np.zeros((n, H, E))
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m['scale'] * w[p + 'temp'][a]
        s = s - w[p + 'r1'][a] * np.log(1.0 + w[p + 'r2'][a] * np.maximum(dist, 0.0))
        s = np.where(vis, s, -np.inf)
        top = np.maximum(s.max(axis=1, keepdims=True), w[p + 'sink'][a])
        e = np.exp(s - top)
        out[:, a] = (e / (e.sum(axis=1, keepdims=True) + np.exp(w[p + 'sink'][a] - top))) @ v[:, g] * gate[:, a:a + 1]
    return out.reshape(n, H * E) @ w[p + 'o'].T


def relu2_feed_forward(h, w, p):
    return np.maximum(h @ w[p + 'up'].T, 0.0) ** 2 @ w[p + 'down'].T


def mixer(kind, h, w, p, m, eps):
    if kind == 'attention':
        return sigmoid_window_attention(h, w, p, m)
    if kind == 'latent_attention':
        return latent_attention(h, w, p, m, eps)
    if kind == 'attention_2':
        return sink_chunk_attention(h, w, p, m, eps)
    raise ValueError(kind)


def hyper_sublayer(xs, fn, w, p):
    """xs [S, n, W] -> new xs: the sublayer reads sum_s in[s] xs[s]; stream t becomes sum_s mix[s, t] xs[s] + out[t] * y."""
    u = np.tensordot(w[p + 'in'], xs, axes=(0, 0))
    y = fn(u)
    return np.tensordot(w[p + 'mix'].T, xs, axes=(1, 0)) + w[p + 'out'][:, None, None] * y[None]


def forward(cfg, w, tokens):
    """tokens [n] -> (logits [n, V], [layer outputs [n, W]]): one sequence from position 0.  Without 'streams' in cfg the
    residual is the plain sum."""
    w = {k: np.asarray(v, np.float64) for k, v in w.items()}
    eps = cfg['norm']['eps']
    x0 = w['embed'][np.asarray(tokens)] * cfg['embedding']['scale']
    S = int(cfg.get('streams') or 0)
    xs = np.stack([x0] * max(S, 1))
    taps = []
    for i, layer in enumerate(cfg['layers']):
        p = f'l{i}.'
        subs = [(1, lambda u, p=p, layer=layer: mixer(layer['type'], offset_rms_norm(u, w[p + 'norm1'], eps), w, p + 'mix.',
                                                       layer['mixer'], eps))]
        if layer.get('mlp'):
            subs.append((2, lambda u, p=p: relu2_feed_forward(offset_rms_norm(u, w[p + 'norm2'], eps), w, p + 'mlp.')))
        for q, fn in subs:
            if S:
                xs = hyper_sublayer(xs, fn, w, f'{p}hc{q}.')
            else:
                xs = xs + fn(xs[0])[None]
        taps.append(xs.sum(axis=0))
    x = xs.sum(axis=0)
    return offset_rms_norm(x, w['final.norm'], eps) @ w['head'].T, taps


def logits(tokens, w, cfg):
    return forward(cfg, w, tokens)[0]


def greedy(prompt, w, cfg, n_new):
    """n_new tokens by arg-max, every one from a whole-sequence pass."""
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(np.argmax(logits(toks, w, cfg)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out
