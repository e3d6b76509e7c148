"""CPU restatement of the reference's gated-DeltaNet decode step.
TEST INFRASTRUCTURE ONLY: imported by tests/; the product never imports it.

Follows the reference's CPU mirror of the DeltaNet block (src/main.cpp:1704-1768), statement by
statement, with its mix of double sums and float products:
  ab     :1704-1714   g = a * softplus(alpha . x + dt_bias), beta = sigmoid(beta_w . x)
  conv   :1715-1732   conv(4) + SiLU + window shift; q / k heads times 1 / max(|head|, eps)
  step   :1733-1755   decay, sk, d, S update, o (row-major S[h][j][i]); kh = h % hK, or h / kdiv
                      (shaders/dn_step.comp:7-10)
  gate   :1756-1767   o / sqrt(mean o^2 + eps) * norm_w * silu(z)

Pinned in tests/test_deltanet_oracle.py: zero state and beta = 1 give S = k (x) v-row outer
product and o = v (q.k) / sqrt(dS); decay alone scales the state; a second write with the same
unit key replaces the stored value (the delta rule's fixed point); the state update equals the
matrix form S*decay + (beta (v - decay S k)) k^T evaluated with numpy; conv of a constant window,
shift order, unit length of q / k heads; softplus limits; both head pairings."""
import numpy as np

F = np.float32


def ab(x, alpha_w, beta_w, dt_bias, a_vec):
    da = alpha_w.astype(np.float64) @ x.astype(np.float64)
    db = beta_w.astype(np.float64) @ x.astype(np.float64)
    v = da + dt_bias.astype(np.float64)
    sp = np.where(v > 20.0, v, np.log1p(np.exp(np.minimum(v, 20.0))))
    return (a_vec.astype(np.float64) * sp).astype(F), (1.0 / (1.0 + np.exp(-db))).astype(F)


def conv(st, qkv, ker, d_state, qk_channels, eps=1e-6):
    """st [channels][3] (updated in place), qkv [channels], ker [channels][4] -> out [channels]."""
    v = (st[:, 0].astype(np.float64) * ker[:, 0] + st[:, 1].astype(np.float64) * ker[:, 1] +
         st[:, 2].astype(np.float64) * ker[:, 2] + qkv.astype(np.float64) * ker[:, 3])
    out = (v / (1.0 + np.exp(-v))).astype(F)
    st[:, 0], st[:, 1], st[:, 2] = st[:, 1].copy(), st[:, 2].copy(), qkv
    for w in range(qk_channels // d_state):
        head = out[w * d_state:(w + 1) * d_state]
        sc = 1.0 / max(np.sqrt((head.astype(np.float64) ** 2).sum()), float(eps))
        head *= F(sc)
    return out


def step(conv_out, g, beta, S, norm_w, z, hK, hV, kdiv=0, eps=1e-6):
    """S [hV][dS][dS] row-major (row j, column i), updated in place.  Returns att [hV*dS]."""
    dS = S.shape[1]
    o = np.empty((hV, dS), dtype=F)
    qsc = F(1.0) / np.sqrt(F(dS))
    for h in range(hV):
        kh = h // kdiv if kdiv else h % hK
        q = conv_out[kh * dS:(kh + 1) * dS]
        k = conv_out[(hK + kh) * dS:(hK + kh + 1) * dS]
        v = conv_out[(2 * hK + h) * dS:(2 * hK + h + 1) * dS]
        decay = np.exp(F(g[h])).astype(F)
        sk = (S[h].astype(np.float64) @ k.astype(np.float64)) * float(decay)
        dj = (F(beta[h]) * (v - sk.astype(F))).astype(F)
        sn = (S[h] * decay + k[None, :] * dj[:, None]).astype(F)
        S[h] = sn
        o[h] = (sn.astype(np.float64) @ (q * qsc).astype(np.float64)).astype(F)
    att = np.empty((hV, dS), dtype=F)
    for h in range(hV):
        sc = 1.0 / np.sqrt((o[h].astype(np.float64) ** 2).sum() / dS + eps)
        zv = z[h * dS:(h + 1) * dS].astype(np.float64)
        att[h] = (o[h].astype(np.float64) * sc * norm_w.astype(np.float64) * (zv / (1.0 + np.exp(-zv)))).astype(F)
    return att.reshape(-1)
