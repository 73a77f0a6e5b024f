"""CPU oracle for the element-wise decoder-layer kernels (TEST INFRASTRUCTURE ONLY).

A numpy restatement of the instruction sequences trueno-gpu's PTX builder describes; only tests/,
__graft_entry__.smoke() and bench.py may import it.

Reference lines followed (under trueno-gpu/src/kernels/):
  residual_add            elementwise.rs:33-101    add.f32
  fused_swiglu            elementwise.rs:521-592   sub, mul by 1.442695f, ex2.approx, add, div.rn, mul, mul
  rmsnorm                 layernorm.rs:388-516     32 lanes, fma per element, shfl.down tree, div.rn, add, rsqrt.approx, mul, mul
  fused_residual_rmsnorm  elementwise.rs:109-248   the same on x = residual + input
  gemv_warp_reduce        gemv.rs:21-166           y[n] = sum_k A[k][n] x[k], A K x N row-major; lane t of 32 takes
                                                   k = t, t+32, ... by fma, then the shfl.down tree
  gemv_coalesced          gemv.rs:188-398          the same product, one thread per column, k in order by fma
  incremental_attention   attention.rs:808-1095    one query per head over a KV cache, online softmax position by position
(div.f32 is printed as div.rn, ex2/rsqrt as .approx: trueno-gpu/src/ptx/builder.rs:1425-1431, 1523-1530.)

Every f32 operation is rounded separately, as the reference's instructions are.  The two approximate
instructions are evaluated exactly here (fp64, rounded to f32); PTX documents them to 2^-22 relative, so the
reference's own outputs lie within that of this oracle, and so must any implementation - that is the tolerance
the tests state.

How each function is pinned (the reference holds no numeric test of these kernels, only names and PTX text):
  residual_add          : exact by definition.
  fused_swiglu          : closed forms (gate = 0 -> 0; large gate -> gate*up; silu(g) - silu(-g) = g), agreement with
                          the fp64 formula gate/(1+exp(-gate))*up (the f32 constant 1.442695 is not log2(e) to the last
                          bit: the difference is covered and bounded in the tests).
  rmsnorm*              : closed forms (constant rows, one-hot rows), mean square of the output, scale invariance,
                          agreement with the fp64 formula; the lane order is an emulation used for error magnitudes.
  gemv_f32_*            : an fp64 matrix product is the closed form; brute force on tiny shapes; the two f32 orders
                          are emulations used for error magnitudes only.
  incremental_attention : fp64 softmax attention is the closed form; special cases (one position; equal keys give the
                          mean of the values; one dominant key gives its value); the position-by-position f32 recurrence
                          is an emulation used for error magnitudes only.
Against a running reference these stay "parity unpinned": it cannot be run here (no Rust, no NVIDIA driver).
"""
import numpy as np

F32 = np.float32
LOG2E_F32 = F32(1.442695)          # the literal of elementwise.rs:570


def residual_add(a, b):
    return (np.asarray(a, F32) + np.asarray(b, F32)).astype(F32)


def fused_swiglu(gate, up):
    """elementwise.rs:565-582, one rounding per instruction, ex2 exact."""
    g = np.asarray(gate, F32)
    u = np.asarray(up, F32)
    neg = (F32(0.0) - g).astype(F32)
    scaled = (neg * LOG2E_F32).astype(F32)
    with np.errstate(over="ignore", under="ignore"):
        e = np.exp2(scaled.astype(np.float64)).astype(F32)
        denom = (F32(1.0) + e).astype(F32)
        sigmoid = (F32(1.0) / denom).astype(F32)
    silu = (g * sigmoid).astype(F32)
    return (silu * u).astype(F32)


def fused_swiglu_fp64(gate, up):
    g = np.asarray(gate, np.float64)
    with np.errstate(over="ignore"):
        return g / (1.0 + np.exp(-g)) * np.asarray(up, np.float64)


def _fma32(a, b, c):
    """fma.rn.f32: the product of two f32 is exact in f64; one further rounding error of 2^-53 relative is far below f32's."""
    return F32(np.float64(a) * np.float64(b) + np.float64(c))


def sum_squares_ref_order(x):
    """layernorm.rs:441-474: lane t of 32 takes elements t, t+32, ... by fma; then shfl.down 16, 8, 4, 2, 1."""
    x = np.asarray(x, F32)
    lanes = np.zeros(32, F32)
    for t in range(32):
        acc = F32(0.0)
        for v in x[t::32]:
            acc = _fma32(v, v, acc)
        lanes[t] = acc
    for d in (16, 8, 4, 2, 1):
        nxt = lanes.copy()
        nxt[:32 - d] = (lanes[:32 - d] + lanes[d:]).astype(F32)
        lanes = nxt
    return lanes[0]


def rmsnorm(x, gamma, eps=1e-5, residual=None):
    """layernorm.rs:476-507 / elementwise.rs:212-240 with the exact reciprocal square root."""
    x = np.asarray(x, F32)
    if residual is not None:
        x = (np.asarray(residual, F32) + x).astype(F32)
    total = sum_squares_ref_order(x)
    mean_sq = F32(total / F32(len(x)))
    rms_inv = F32(1.0 / np.sqrt(np.float64(F32(mean_sq + F32(eps)))))
    return ((x * rms_inv).astype(F32) * np.asarray(gamma, F32)).astype(F32)


def rmsnorm_fp64(x, gamma, eps=1e-5, residual=None):
    x = np.asarray(x, np.float64)
    if residual is not None:
        x = (np.asarray(residual, F32) + np.asarray(x, F32)).astype(np.float64)     # the add is an f32 add in the reference
    return x / np.sqrt(np.mean(x * x) + np.float64(F32(eps))) * np.asarray(gamma, np.float64)


def gemv_f32_fp64(a, x):
    """y[n] = sum_k A[k][n] x[k] (gemv.rs:1-15): A is K x N row-major."""
    return np.asarray(x, np.float64) @ np.asarray(a, np.float64)


def gemv_f32_coalesced_order(a, x):
    """gemv.rs:292-378: per column, sum = fma(x[k], A[k][n], sum) for k = 0, 1, 2, ..."""
    a, x = np.asarray(a, F32), np.asarray(x, F32)
    acc = np.zeros(a.shape[1], F32)
    for k in range(a.shape[0]):
        acc = (np.float64(x[k]) * a[k].astype(np.float64) + acc.astype(np.float64)).astype(F32)
    return acc


def gemv_f32_warp_reduce_order(a, x):
    """gemv.rs:84-132: lane t accumulates k = t, t+32, ... by fma; then shfl.down 16, 8, 4, 2, 1."""
    a, x = np.asarray(a, F32), np.asarray(x, F32)
    lanes = np.zeros((32, a.shape[1]), F32)
    for k in range(a.shape[0]):
        t = k % 32
        lanes[t] = (np.float64(x[k]) * a[k].astype(np.float64) + lanes[t].astype(np.float64)).astype(F32)
    for d in (16, 8, 4, 2, 1):
        nxt = lanes.copy()
        nxt[:32 - d] = (lanes[:32 - d] + lanes[d:]).astype(F32)
        lanes = nxt
    return lanes[0]


def attention_fp64(q, k, v, seq_len, scale=None):
    """out[h] = softmax(scale * q[h] . k[kv(h)][:seq_len]) @ v[kv(h)][:seq_len], kv(h) = h * num_kv_heads // num_heads
    (attention.rs:877-885, 920-922).  q [H][D]; k, v [Hkv][max_seq][D]."""
    q, k, v = (np.asarray(a, np.float64) for a in (q, k, v))
    H, D = q.shape
    Hkv = k.shape[0]
    scale = 1.0 / np.sqrt(D) if scale is None else float(scale)
    out = np.zeros((H, D))
    for h in range(H):
        kv = h * Hkv // H
        s = (k[kv, :seq_len] @ q[h]) * scale
        w = np.exp(s - s.max())
        out[h] = (w / w.sum()) @ v[kv, :seq_len]
    return out


def attention_ref_order(q, k, v, seq_len, scale=None):
    """The reference's recurrence in f32 (attention.rs:963-1066): per position the dot product (lane order ignored:
    summed in f64 and rounded once), score = dot * scale, new max, correction = 2^((old-new)*log2e), e = 2^((score-new)*log2e),
    sum = sum*correction + e, out = out*correction + e*v; finally out * (1/sum).  ex2 evaluated exactly."""
    q, k, v = (np.asarray(a, F32) for a in (q, k, v))
    H, D = q.shape
    Hkv = k.shape[0]
    scale = F32(1.0 / np.sqrt(F32(D))) if scale is None else F32(scale)
    log2e = F32(1.4426950)
    out = np.zeros((H, D), F32)
    with np.errstate(over="ignore", invalid="ignore"):
        for h in range(H):
            kv = h * Hkv // H
            m, ssum, o = F32(-np.inf), F32(0.0), np.zeros(D, F32)
            for p in range(seq_len):
                score = F32(F32(np.dot(q[h].astype(np.float64), k[kv, p].astype(np.float64))) * scale)
                nm = max(m, score)
                corr = F32(np.exp2(np.float64(F32(F32(m - nm) * log2e)))) if np.isfinite(m) else F32(0.0)
                e = F32(np.exp2(np.float64(F32(F32(score - nm) * log2e))))
                ssum = F32(F32(ssum * corr) + e)
                o = ((o * corr).astype(F32).astype(np.float64) + np.float64(e) * v[kv, p].astype(np.float64)).astype(F32)
                m = nm
            out[h] = (o * F32(F32(1.0) / ssum)).astype(F32)
    return out
