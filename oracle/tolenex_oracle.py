"""Plain float64 numpy statement of the Tolenex design, one function per mechanism.  Test infrastructure only: slow, whole
sequences, no cache, no batching - the product (the stack engine) never touches it and shares no code with it.

Notation: n tokens, width W, a layer's mixer has H heads of query/key size D and value size E.  Weights `w` is a dict
name -> float64 array with the checkpoint's names; `cfg` is the parsed config.json."""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def grouped_rms_norm(x, weight, groups, eps):
    """x [..., W] cut into `groups` consecutive parts, each scaled by 1 / sqrt(mean(part^2) + eps); then * weight."""
    parts = x.reshape(x.shape[:-1] + (groups, x.shape[-1] // groups))
    parts = parts / np.sqrt(np.mean(parts * parts, axis=-1, keepdims=True) + eps)
    return parts.reshape(x.shape) * weight


def rotary_frequencies(rot):
    """(frequency per pair [dims / 2], multiplier of cos and sin) with the YaRN blend when rot['scaling'] is there."""
    dims, base = rot['dims'], rot['base']
    i = np.arange(dims // 2, dtype=np.float64)
    freq = base ** (-2.0 * i / dims)
    sc = rot.get('scaling')
    if not sc:
        return freq, 1.0

    def dim_of(turns):
        return dims * math.log(sc['original'] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(sc['fast'])), 0)
    hi = min(math.ceil(dim_of(sc['slow'])), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return freq / sc['factor'] * ramp + freq * (1.0 - ramp), 0.1 * math.log(sc['factor']) + 1.0


def rotate_pairs(x, positions, rot):
    """x [n, heads, D]: dimensions (2i, 2i + 1), i < dims / 2, turn by positions * freq_i; the rest pass."""
    if not rot or not rot.get('dims'):
        return x
    freq, mult = rotary_frequencies(rot)
    dims = rot['dims']
    ang = positions[:, None].astype(np.float64) * freq[None, :]
    c, s = (np.cos(ang) * mult)[:, None, :], (np.sin(ang) * mult)[:, None, :]
    even, odd = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.copy()
    out[..., 0:dims:2] = even * c - odd * s
    out[..., 1:dims:2] = odd * c + even * s
    return out


def differential_attention(h, w, prefix, mixer, eps):
    """h [n, W] -> [n, W].  Two softmax maps per head over shared values, o = a1 - lam * a2, unit RMS per head, * (1 - diff)."""
    n = h.shape[0]
    H, G, D, E = mixer['heads'], mixer.get('kv_heads', mixer['heads']), mixer['dim'], mixer.get('vdim', mixer['dim'])
    pos = np.arange(n)
    q = rotate_pairs((h @ w[prefix + 'mix.q'].T).reshape(n, H * 2, D), pos, mixer.get('rot')).reshape(n, H, 2, D)
    k = rotate_pairs((h @ w[prefix + 'mix.k'].T).reshape(n, G * 2, D), pos, mixer.get('rot')).reshape(n, G, 2, D)
    v = (h @ w[prefix + 'mix.v'].T).reshape(n, G, E)
    lam = (math.exp(float(np.sum(w[prefix + 'mix.lq1'] * w[prefix + 'mix.lk1'])))
           - math.exp(float(np.sum(w[prefix + 'mix.lq2'] * w[prefix + 'mix.lk2']))) + mixer['diff'])
    cap = mixer.get('softcap') or 0.0
    visible = np.tril(np.ones((n, n), bool))
    heads = []
    for head in range(H):
        g = head // (H // G)
        maps = []
        for m in range(2):
            s = (q[:, head, m] @ k[:, g, m].T) * mixer['scale']
            if cap:
                s = cap * np.tanh(s / cap)
            s = np.where(visible, s, -np.inf)
            p = np.exp(s - s.max(axis=1, keepdims=True))
            maps.append((p / p.sum(axis=1, keepdims=True)) @ v[:, g])
        o = maps[0] - lam * maps[1]
        heads.append(o / np.sqrt(np.mean(o * o, axis=1, keepdims=True) + eps) * (1.0 - mixer['diff']))
    return np.concatenate(heads, axis=1) @ w[prefix + 'mix.o'].T


def hgrn2_mixer(h, w, prefix, mixer, eps):
    """h [n, W] -> [n, W].  S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T per head (S [D, E], zero at the start), o_t = S_t^T q_t."""
    n = h.shape[0]
    H, D, E = mixer['heads'], mixer['dim'], mixer.get('vdim', mixer['dim'])
    z = h @ w[prefix + 'mix.q'].T
    q = (z * sigmoid(z)).reshape(n, H, D)
    v = (h @ w[prefix + 'mix.v'].T).reshape(n, H, E)
    low = w[prefix + 'mix.lower']
    f = (low + (1.0 - low) * sigmoid(h @ w[prefix + 'mix.f'].T + w[prefix + 'mix.f.b'])).reshape(n, H, D)
    S = np.zeros((H, D, E))
    out = np.zeros((n, H, E))
    for t in range(n):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = np.einsum('hde,hd->he', S, q[t])
    out = out / np.sqrt(np.mean(out * out, axis=2, keepdims=True) + eps) * w[prefix + 'mix.norm']
    return out.reshape(n, H * E) @ w[prefix + 'mix.o'].T


def gated_mlp(h, w, prefix):
    return (gelu_tanh(h @ w[prefix + 'mlp.gate'].T) * (h @ w[prefix + 'mlp.up'].T)) @ w[prefix + 'mlp.down'].T


def layer_order(cfg):
    """[(layer index, pass number when the layer opens a pass of the loop, else None)] in execution order."""
    L = len(cfg['layers'])
    loop = cfg.get('loop')
    if not loop or loop['stop'] <= loop['start']:
        return [(i, None) for i in range(L)]
    order = [(i, None) for i in range(loop['start'])]
    for t in range(loop['times']):
        order += [(i, t if i == loop['start'] else None) for i in range(loop['start'], loop['stop'])]
    return order + [(i, None) for i in range(loop['stop'], L)]


def tolenex_logits(tokens, w, cfg, residuals=None):
    """tokens [n] -> logits [n, vocab] (float64).  residuals: optional list that receives x behind every layer run."""
    eps, groups = cfg['norm']['eps'], cfg['norm']['groups']
    emb = w['embed'][np.asarray(tokens)] * cfg['embedding']['scale']
    x = emb.copy()
    for i, opens in layer_order(cfg):
        if opens is not None:
            if opens > 0:
                x = x + emb
            x = x + w['loop.step'][opens]
        layer, p = cfg['layers'][i], f'l{i}.'
        h1 = grouped_rms_norm(x, w[p + 'norm1'], groups, eps)
        mix = differential_attention if layer['type'] == 'attention' else hgrn2_mixer
        update = mix(h1, w, p, layer['mixer'], eps) * sigmoid(h1 @ w[p + 'rg1'].T + w[p + 'rg1.b'])
        if layer.get('mlp'):
            h2 = grouped_rms_norm(x, w[p + 'norm2'], groups, eps)
            update = update + gated_mlp(h2, w, p) * sigmoid(h2 @ w[p + 'rg2'].T + w[p + 'rg2.b'])
        x = x + update
        if residuals is not None:
            residuals.append(x.copy())
    return grouped_rms_norm(x, w['final.norm'], groups, eps) @ w['head'].T


def greedy(tokens, w, cfg, new_tokens):
    """Greedy continuation by recomputing the whole sequence for every token."""
    seq = list(tokens)
    for _ in range(new_tokens):
        seq.append(int(np.argmax(tolenex_logits(seq, w, cfg)[-1])))
    return seq[len(tokens):]
