"""
CPU oracle (TEST INFRASTRUCTURE, not product code).

A numpy restatement of the numpy checks the reference ships for its compute
core, plus closed-form definitions of the pieces the reference only defines in
device code (rounding, stochastic rounding, integer saturation).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module.  The product package must never route through it.

Each function cites the reference file:line it follows (paths are relative to
the reference checkout).

Pinning status (what independent check fixes each function; see
tests/test_oracle_*.py):

  ref_dot / ref_batched_dot      np.dot in float64 (library routine); all-ones
                                 known answer C == k (benchmarks/gemm_test2.py:40-41,
                                 kernels/C_interface/test.cu:42-51).
  ref_conv_fprop/bprop/update    brute-force nested loops on tiny shapes, torch CPU
                                 conv2d/conv3d (+autograd), adjoint identity.
  ref_pool_*                     torch CPU max_pool/avg_pool (+autograd), brute force
                                 for J>1 and padded windows, adjoint identity for avg.
  f32_to_f16_rz / round_*        exhaustive comparison with numpy's own float16 cast
                                 on exactly representable values, bracket/expectation
                                 invariants for stochastic rounding.
  rand32                         bijectivity in idx on 2^16 windows, hard-coded
                                 known-answer vectors (golden fixture).
  magic32                        exhaustive n//d == (n*m)>>s.
  ref_ew                         numpy expression evaluated directly in the tests.
  ref_compensated_sum            Kahan closed form: sum+cmp tracks the fp64 sum.
"""
import numpy as np

__all__ = [
    "contiguous_strides", "magic32", "fast_ew_dims", "gemm_tile_heuristic",
    "rand32", "rand_sr16", "rand_uniform", "f32_to_f16_rz", "round_fp16_rn", "round_int",
    "round_stochastic_fp16", "round_stochastic_fp32", "round_store",
    "ref_dot", "ref_batched_dot",
    "conv_out_dims", "conv_pixel_indices", "ref_conv_fprop", "ref_conv_bprop",
    "ref_conv_update", "ref_conv_fprop_pixels", "ref_conv_bprop_pixels",
    "ref_conv_update_rows",
    "pool_out_dims", "pool_pixel_indices", "ref_pool_fprop", "ref_pool_bprop",
    "ref_pool_fprop_pixels",
    "ref_ew", "ref_transpose", "ref_dimshuffle", "ref_compensated_sum",
    "ref_batchnorm_rows",
]


# --------------------------------------------------------------------------
# small host helpers
# --------------------------------------------------------------------------

def contiguous_strides(shape):
    """Row-major element strides (nervanagpu/nervanagpu.py:1324-1331)."""
    if not shape:
        return ()
    strides = [1]
    for s in shape[:0:-1]:
        strides.append(strides[-1] * s)
    return tuple(strides[::-1])


def magic32(nmax, d):
    """(magic, shift) with n//d == (n*magic)>>shift for 0<=n<=nmax
    (nervanagpu/layers.py:761-768)."""
    nc = ((nmax + 1) // d) * d - 1
    nbits = len(bin(nmax)) - 2
    for p in range(0, 2 * nbits + 1):
        if 2 ** p > nc * (d - 1 - (2 ** p - 1) % d):
            m = (2 ** p + d - 1 - (2 ** p - 1) % d) // d
            return (m, p)
    raise ValueError("Can't find magic number for division")


def fast_ew_dims(size):
    """2-D view used for plain contiguous elementwise ops
    (nervanagpu/float_ew.py:1037-1055)."""
    ew_size = 256
    while ew_size > 0:
        if size % ew_size == 0:
            break
        ew_size -= 32
    if ew_size == 0:
        ew_size = 255
        while ew_size > 0:
            if size % ew_size == 0:
                break
            ew_size -= 1
    shape = (size // ew_size, ew_size)
    return shape, contiguous_strides(shape)


def gemm_tile_heuristic(op, m, n, sm_count):
    """Advisory tile choice of the reference (nervanagpu/nervanagpu.py:1007-1047,
    duplicated in kernels/C_interface/nervana_c_api.cu:132-202).  Returns "AxB"."""
    short = min(m, n)
    if short < 384 - 16:
        short128 = short % 128
        if 0 < short128 < 112:
            if 48 < short128 <= 64:
                occupancy64 = short // 64
                wide = max(m, n)
                occupancy64 *= (wide // 128 + (wide % 128 != 0)) // sm_count
                size = 64 if occupancy64 > 1 else 32
            else:
                size = 32
        else:
            size = 128
    else:
        size = 128
    if m >= n:
        if op == "nt":
            size = 128
        return "%dx%d" % (128, size)
    if op == "tn":
        size = 128
    elif size == 64:
        size = 32
    return "%dx%d" % (size, 128)


# --------------------------------------------------------------------------
# counter-based random stream and rounding
# --------------------------------------------------------------------------
# The reference's generator (a Tausworthe LFSR re-seeded from the SM clock,
# nervanagpu/float_ew.py:113-144) is irreproducible by construction.  The build
# keeps the *meaning* of its stochastic rounding (float_ew.py:126-130, 182-201)
# and replaces the stream by a stateless hash of (seed, stream, element index).

_U32 = np.uint32


def _fmix32_scalar(h):
    h &= 0xFFFFFFFF
    h ^= h >> 16
    h = (h * 0x85EBCA6B) & 0xFFFFFFFF
    h ^= h >> 13
    h = (h * 0xC2B2AE35) & 0xFFFFFFFF
    h ^= h >> 16
    return h


def rand32(seed, stream, idx):
    """32 random bits for element `idx` of launch `stream` under `seed`.
    Two keys derived from (seed, stream) with the murmur3 finaliser, then a
    two-multiply integer hash of idx; a bijection of idx for fixed keys, so a
    full sweep of idx is exactly uniform."""
    seed = int(seed) & 0xFFFFFFFF
    stream = int(stream) & 0xFFFFFFFF
    ka = (_fmix32_scalar(seed ^ 0x9E3779B9) + stream * 0x85EBCA77) & 0xFFFFFFFF
    kb = _fmix32_scalar((stream + 0xC2B2AE3D) & 0xFFFFFFFF) ^ seed
    with np.errstate(over="ignore"):
        x = np.asarray(idx).astype(np.uint32) + _U32(ka)
        x ^= x >> _U32(16)
        x *= _U32(0x7FEB352D)
        x ^= _U32(kb)
        x ^= x >> _U32(15)
        x *= _U32(0x846CA68B)
        x ^= x >> _U32(16)
    return x


def rand_sr16(seed, stream, idx):
    """Random word for the fp16 stochastic rounding of element `idx`: elements
    2i and 2i+1 share the draw of index i (fp16 needs at most 16 random bits);
    the even element uses the high half, the odd one the low half."""
    idx = np.asarray(idx).astype(np.uint32)
    h = rand32(seed, stream, idx >> _U32(1))
    return np.where((idx & _U32(1)) != 0, h << _U32(16), h).astype(np.uint32)


def rand_uniform(seed, stream, idx):
    """The `rand` op: RN convert of 32 random bits times 2^-32, in [0, 1]
    (nervanagpu/float_ew.py:146-155)."""
    return rand32(seed, stream, idx).astype(np.float32) * np.float32(2.0 ** -32)


def f32_to_f16_rz(x):
    """fp32 -> fp16 bit patterns (uint16) with round-toward-zero: overflow
    saturates at 65504, subnormal results are truncated
    (cvt.rz.f16.f32, nervanagpu/float_ew.py:196)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    sign = ((u >> _U32(16)) & _U32(0x8000)).astype(np.uint32)
    mag = u & _U32(0x7FFFFFFF)
    exp = (mag >> _U32(23)).astype(np.int32)
    man = mag & _U32(0x7FFFFF)
    # normal fp16 range
    normal = (((exp - 112).astype(np.uint32) << _U32(10)) | (man >> _U32(13)))
    # subnormal fp16: value / 2^-24, truncated
    shift = np.clip(126 - exp, 0, 31).astype(np.uint32)  # 14 for e=-15 ... 24 for e=-25
    sub = np.where(shift >= 24 + 1, _U32(0), (man | _U32(0x800000)) >> shift)
    h = np.where(exp >= 113, normal, sub)
    h = np.where(exp < 102, _U32(0), h)                    # |x| < 2^-25 -> 0
    h = np.where(mag >= _U32(0x47800000), _U32(0x7BFF), h)  # >= 65536 -> max finite
    h = np.where(mag == _U32(0x7F800000), _U32(0x7C00), h)  # inf
    h = np.where(mag > _U32(0x7F800000), _U32(0x7E00), h)   # nan
    return (h | sign).astype(np.uint16)


def round_fp16_rn(x):
    """cvt.rn.f16.f32 (nervanagpu/float_ew.py:257-267): round-to-nearest-even."""
    return np.asarray(x, dtype=np.float32).astype(np.float16)


def round_int(x, dtype):
    """cvt.rni.<int>.f32 (nervanagpu/float_ew.py:269-316): round-half-even and
    saturate; the host-side statement is np.around + clip
    (nervanagpu/tests/test_tensor.py:50-53)."""
    info = np.iinfo(dtype)
    x = np.asarray(x, dtype=np.float32)
    r = np.around(np.nan_to_num(x.astype(np.float64), nan=0.0,
                                posinf=float(info.max), neginf=float(info.min)))
    return np.clip(r, info.min, info.max).astype(dtype)


def _sr_bits(x, bits, r, clamp_mag=None):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = np.asarray(r).astype(np.uint32)
    d = 23 - int(bits)
    assert 1 <= bits <= 22
    mask = _U32((0xFFFFFFFF << d) & 0xFFFFFFFF)
    sign = u & _U32(0x80000000)
    mag = u & _U32(0x7FFFFFFF)
    finite = mag < _U32(0x7F800000)
    base = mag if clamp_mag is None else np.minimum(mag, _U32(clamp_mag))
    with np.errstate(over="ignore"):
        m2 = (base + (r >> _U32(32 - d))) & mask
    m2 = np.where(m2 >= _U32(0x7F800000), _U32(0x7F7FFFFF) & mask, m2)
    m2 = np.where(finite, m2, mag)
    return (sign | m2).astype(np.uint32)


def round_stochastic_fp32(x, bits, r):
    """fp32 value truncated to `bits` mantissa bits after adding a uniform
    fraction of one unit at that precision to the magnitude
    (fp32_to_fp32_rand, nervanagpu/float_ew.py:162-180)."""
    return _sr_bits(x, bits, r).view(np.float32)


def round_stochastic_fp16(x, bits, r):
    """fp32 -> fp16 (returned as float16) with stochastic rounding at `bits`
    (<=10) mantissa bits (fp32_to_fp16_rand, nervanagpu/float_ew.py:182-201)."""
    # finite magnitudes saturate at the largest fp16 value (65504 = 0x477FE000)
    # before the random increment, so it can never carry into infinity
    v = _sr_bits(x, min(int(bits), 10), r, clamp_mag=0x477FE000).view(np.float32)
    return f32_to_f16_rz(v).view(np.float16)


def round_store(x32, dtype, rounding=0, r=None):
    """The store step of every kernel: fp32 register value -> storage dtype.
    rounding: 0 = nearest; else mantissa bits for fp16/fp32 stochastic rounding
    (clamps as in nervanagpu/float_ew.py:1227-1237).  Integer outputs are always
    round-half-even + saturate (the reference's int SR strings never compiled,
    float_ew.py:438-440)."""
    dtype = np.dtype(dtype)
    x32 = np.asarray(x32, dtype=np.float32)
    if dtype == np.float32:
        if rounding:
            return round_stochastic_fp32(x32, max(min(int(rounding), 15), 1), r)
        return x32
    if dtype == np.float16:
        if rounding:
            return round_stochastic_fp16(x32, max(min(int(rounding), 10), 1), r)
        return round_fp16_rn(x32)
    return round_int(x32, dtype)


# --------------------------------------------------------------------------
# GEMM
# --------------------------------------------------------------------------

def ref_dot(A, B, C=None, alpha=1.0, beta=0.0, relu=False, acc_dtype=np.float64):
    """fp32 pre-rounding value of C = beta*C + relu(alpha * A.B)
    (np.dot check: benchmarks/gemm_test.py:59; epilogue order alpha -> relu ->
    +beta*C: kernels/sass/hgemm_common_128x128.sass:183-264).
    A and B are the already transposed logical operands (m,k) and (k,n)."""
    acc = np.dot(np.asarray(A, dtype=acc_dtype), np.asarray(B, dtype=acc_dtype))
    acc = acc * acc_dtype(alpha)
    if relu:
        acc = np.maximum(acc, 0)
    if beta != 0.0:
        acc = acc + acc_dtype(beta) * np.asarray(C, dtype=acc_dtype)
    return acc.astype(np.float32)


def ref_batched_dot(A, B, C=None, alpha=1.0, beta=0.0, relu=False, out_3d=True,
                    acc_dtype=np.float64):
    """batched_dot (nervanagpu/nervanagpu.py:820-957; numpy check
    benchmarks/batched_dot_test.py:65-74).  A and/or B are 3-D (batch,.,.); a
    2-D operand is broadcast.  out_3d=True: one GEMM per batch; False: the
    products are summed over the batch into a single 2-D C."""
    A = np.asarray(A, dtype=acc_dtype)
    B = np.asarray(B, dtype=acc_dtype)
    nb = A.shape[0] if A.ndim == 3 else B.shape[0]
    prods = []
    for b in range(nb):
        a = A[b] if A.ndim == 3 else A
        bb = B[b] if B.ndim == 3 else B
        prods.append(np.dot(a, bb))
    if out_3d:
        acc = np.stack(prods) * acc_dtype(alpha)
    else:
        acc = np.sum(np.stack(prods), axis=0) * acc_dtype(alpha)
    if relu:
        acc = np.maximum(acc, 0)
    if beta != 0.0:
        acc = acc + acc_dtype(beta) * np.asarray(C, dtype=acc_dtype)
    return acc.astype(np.float32)


# --------------------------------------------------------------------------
# convolution (CHWN, filters CTRSK, outputs KMPQN)
# --------------------------------------------------------------------------

def _ceil_div(a, b):
    return -(-a // b)


def conv_out_dims(DHW, TRS, padding, strides):
    """M,P,Q = ceil((D - T + 1 + 2*pad)/stride) (nervanagpu/layers.py:297-301)."""
    return tuple(_ceil_div(d - t + 1 + 2 * p, s)
                 for d, t, p, s in zip(DHW, TRS, padding, strides))


def conv_pixel_indices(C, DHW, TRS, mt, pr, qs):
    """Flat (c,z,y,x) row indices of the receptive field of one output pixel,
    out-of-bounds taps pointing at the extra zero row C*D*H*W
    (benchmarks/conv_test.py:99-130)."""
    T, R, S = TRS
    D, H, W = DHW
    HW = H * W
    DHWs = D * HW
    imax = C * DHWs
    t = np.arange(T)[:, None, None]
    r = np.arange(R)[None, :, None]
    s = np.arange(S)[None, None, :]
    z, y, x = mt + t, pr + r, qs + s
    ok = (z >= 0) & (z < D) & (y >= 0) & (y < H) & (x >= 0) & (x < W)
    sp = z * HW + y * W + x
    c = np.arange(C)[:, None, None, None] * DHWs
    idx = np.where(ok[None], c + sp[None], imax)
    return idx.reshape(-1)


def _slicable(a, pad_value=None):
    """collapse outer dims, keep N; optionally append one padding row
    (benchmarks/conv_test.py:47-50, 66-67)."""
    a2 = a.reshape(-1, a.shape[-1])
    if pad_value is None:
        return a2
    row = np.full((1, a2.shape[1]), pad_value, dtype=a2.dtype)
    return np.concatenate([a2, row], axis=0)


def _conv_setup(I_shape, F_shape, padding, strides):
    C, D, H, W, N = I_shape
    C2, T, R, S, K = F_shape
    assert C == C2
    MPQ = conv_out_dims((D, H, W), (T, R, S), padding, strides)
    return C, (D, H, W), (T, R, S), K, N, MPQ


def ref_conv_fprop(I, F, padding=(0, 0, 0), strides=(1, 1, 1), alpha=1.0,
                   relu=False, acc_dtype=np.float64):
    """O[:,m,p,q,:] = F.T . I[idx,:] per output pixel
    (benchmarks/conv_test.py:138-158).  Returns the fp32 pre-rounding value."""
    C, DHW, TRS, K, N, (M, P, Q) = _conv_setup(I.shape, F.shape, padding, strides)
    I2 = _slicable(np.asarray(I, dtype=acc_dtype), 0)
    Ft = np.ascontiguousarray(np.asarray(F, dtype=acc_dtype).reshape(-1, K).T)
    O = np.zeros((K, M, P, Q, N), dtype=acc_dtype)
    for m in range(M):
        mt = m * strides[0] - padding[0]
        for p in range(P):
            pr = p * strides[1] - padding[1]
            for q in range(Q):
                qs = q * strides[2] - padding[2]
                idx = conv_pixel_indices(C, DHW, TRS, mt, pr, qs)
                O[:, m, p, q, :] = np.dot(Ft, I2[idx, :])
    O *= alpha
    if relu:
        O = np.maximum(O, 0)
    return O.astype(np.float32)


def ref_conv_bprop(F, E, I_shape, padding=(0, 0, 0), strides=(1, 1, 1), alpha=1.0,
                   acc_dtype=np.float64):
    """gradI[idx,:] += F . E[:,m,p,q,:] per output pixel
    (benchmarks/conv_test.py:160-161)."""
    C, DHW, TRS, K, N, (M, P, Q) = _conv_setup(I_shape, F.shape, padding, strides)
    F2 = np.asarray(F, dtype=acc_dtype).reshape(-1, K)
    E = np.asarray(E, dtype=acc_dtype)
    B = np.zeros((C * DHW[0] * DHW[1] * DHW[2] + 1, N), dtype=acc_dtype)
    for m in range(M):
        mt = m * strides[0] - padding[0]
        for p in range(P):
            pr = p * strides[1] - padding[1]
            for q in range(Q):
                qs = q * strides[2] - padding[2]
                idx = conv_pixel_indices(C, DHW, TRS, mt, pr, qs)
                B[idx, :] += np.dot(F2, E[:, m, p, q, :])
    return (B[:-1] * alpha).reshape(I_shape).astype(np.float32)


def ref_conv_update(I, E, F_shape, padding=(0, 0, 0), strides=(1, 1, 1), alpha=1.0,
                    acc_dtype=np.float64):
    """gradF += I[idx,:] . E[:,m,p,q,:].T per output pixel
    (benchmarks/conv_test.py:163-164)."""
    C, DHW, TRS, K, N, (M, P, Q) = _conv_setup(I.shape, F_shape, padding, strides)
    I2 = _slicable(np.asarray(I, dtype=acc_dtype), 0)
    E = np.asarray(E, dtype=acc_dtype)
    U = np.zeros((C * TRS[0] * TRS[1] * TRS[2], K), dtype=acc_dtype)
    for m in range(M):
        mt = m * strides[0] - padding[0]
        for p in range(P):
            pr = p * strides[1] - padding[1]
            for q in range(Q):
                qs = q * strides[2] - padding[2]
                idx = conv_pixel_indices(C, DHW, TRS, mt, pr, qs)
                U += np.dot(I2[idx, :], E[:, m, p, q, :].T)
    return (U * alpha).reshape(F_shape).astype(np.float32)


def ref_conv_fprop_pixels(I, F, pixels, padding=(0, 0, 0), strides=(1, 1, 1),
                          alpha=1.0, relu=False, acc_dtype=np.float64):
    """ref_conv_fprop restricted to a list of output pixels (m,p,q);
    returns (len(pixels), K, N).  Same per-pixel statement as
    benchmarks/conv_test.py:155-158; used to spot-check full-size layers."""
    C, DHW, TRS, K, N, _ = _conv_setup(I.shape, F.shape, padding, strides)
    I2 = I.reshape(-1, N)
    Ft = np.ascontiguousarray(np.asarray(F, dtype=acc_dtype).reshape(-1, K).T)
    out = np.zeros((len(pixels), K, N), dtype=acc_dtype)
    imax = I2.shape[0]
    for i, (m, p, q) in enumerate(pixels):
        idx = conv_pixel_indices(C, DHW, TRS, m * strides[0] - padding[0],
                                 p * strides[1] - padding[1], q * strides[2] - padding[2])
        ok = idx < imax
        rows = np.zeros((idx.size, N), dtype=acc_dtype)
        rows[ok] = I2[idx[ok]]
        out[i] = np.dot(Ft, rows)
    out *= alpha
    if relu:
        out = np.maximum(out, 0)
    return out.astype(np.float32)


def ref_conv_bprop_pixels(F, E, I_shape, pixels, padding=(0, 0, 0), strides=(1, 1, 1),
                          alpha=1.0, acc_dtype=np.float64):
    """gradI[:, z,y,x, :] for a list of input pixels (z,y,x), in gather form:
    the sum over every (output pixel, tap) pair whose receptive field touches
    the input pixel.  Adjoint of benchmarks/conv_test.py:155-158; pinned against
    ref_conv_bprop in the oracle tests.  Returns (len(pixels), C, N)."""
    C, DHW, TRS, K, N, (M, P, Q) = _conv_setup(I_shape, F.shape, padding, strides)
    T, R, S = TRS
    F5 = np.asarray(F, dtype=acc_dtype)
    out = np.zeros((len(pixels), C, N), dtype=acc_dtype)
    for i, (z, y, x) in enumerate(pixels):
        for t in range(T):
            mz = z + padding[0] - t
            if mz % strides[0] or not (0 <= mz // strides[0] < M):
                continue
            for r in range(R):
                py = y + padding[1] - r
                if py % strides[1] or not (0 <= py // strides[1] < P):
                    continue
                for s in range(S):
                    qx = x + padding[2] - s
                    if qx % strides[2] or not (0 <= qx // strides[2] < Q):
                        continue
                    e = np.asarray(E[:, mz // strides[0], py // strides[1], qx // strides[2], :],
                                   dtype=acc_dtype)
                    out[i] += np.dot(F5[:, t, r, s, :], e)
    return (out * alpha).astype(np.float32)


def ref_conv_update_rows(I, E, F_shape, rows, padding=(0, 0, 0), strides=(1, 1, 1),
                         alpha=1.0, acc_dtype=np.float64):
    """ref_conv_update restricted to a list of flat (c,t,r,s) filter rows;
    returns (len(rows), K)."""
    C, DHW, TRS, K, N, (M, P, Q) = _conv_setup(I.shape, F_shape, padding, strides)
    I2 = I.reshape(-1, N)
    imax = I2.shape[0]
    rows = np.asarray(rows)
    U = np.zeros((rows.size, K), dtype=acc_dtype)
    for m in range(M):
        for p in range(P):
            for q in range(Q):
                idx = conv_pixel_indices(C, DHW, TRS, m * strides[0] - padding[0],
                                         p * strides[1] - padding[1],
                                         q * strides[2] - padding[2])[rows]
                ok = idx < imax
                if not ok.any():
                    continue
                g = np.zeros((rows.size, N), dtype=acc_dtype)
                g[ok] = I2[idx[ok]]
                U += np.dot(g, np.asarray(E[:, m, p, q, :], dtype=acc_dtype).T)
    return (U * alpha).astype(np.float32)


# --------------------------------------------------------------------------
# pooling (window J over channels, T,R,S over space)
# --------------------------------------------------------------------------

def pool_out_dims(CDHW, JTRS, padding, strides):
    """K,M,P,Q (nervanagpu/layers.py:566-569)."""
    return tuple(_ceil_div(d - w + 1 + 2 * p, s)
                 for d, w, p, s in zip(CDHW, JTRS, padding, strides))


def pool_pixel_indices(C, DHW, JTRS, kj, mt, pr, qs):
    """Flat row indices of one pooling window in (j,t,r,s) scan order,
    out-of-bounds slots pointing at the extra row C*D*H*W
    (benchmarks/pool_test.py:71-104)."""
    J, T, R, S = JTRS
    D, H, W = DHW
    HW = H * W
    DHWs = D * HW
    imax = C * DHWs
    j = np.arange(J)[:, None, None, None]
    t = np.arange(T)[None, :, None, None]
    r = np.arange(R)[None, None, :, None]
    s = np.arange(S)[None, None, None, :]
    c, z, y, x = kj + j, mt + t, pr + r, qs + s
    ok = ((c >= 0) & (c < C) & (z >= 0) & (z < D) & (y >= 0) & (y < H)
          & (x >= 0) & (x < W))
    idx = np.where(ok, c * DHWs + z * HW + y * W + x, imax)
    return idx.reshape(-1)


def _pool_setup(I_shape, JTRS, padding, strides):
    C, D, H, W, N = I_shape
    if strides is None:
        strides = JTRS
    KMPQ = pool_out_dims((C, D, H, W), JTRS, padding, strides)
    return C, (D, H, W), N, tuple(strides), KMPQ


def _pool_windows(C, DHW, JTRS, padding, strides, KMPQ):
    K, M, P, Q = KMPQ
    for k in range(K):
        kj = k * strides[0] - padding[0]
        for m in range(M):
            mt = m * strides[1] - padding[1]
            for p in range(P):
                pr = p * strides[2] - padding[2]
                for q in range(Q):
                    qs = q * strides[3] - padding[3]
                    yield (k, m, p, q), pool_pixel_indices(C, DHW, JTRS, kj, mt, pr, qs)


def ref_pool_fprop(I, op, JTRS, padding=(0, 0, 0, 0), strides=None):
    """max: np.max over the window with out-of-bounds slots = -FLT_MAX;
    avg: np.mean over all J*T*R*S slots with out-of-bounds slots = 0;
    l2: sqrt of the sum of squares over the window, out-of-bounds slots = 0
    (benchmarks/pool_test.py:38-42, 120-146).  fp32 pre-rounding value."""
    C, DHW, N, strides, KMPQ = _pool_setup(I.shape, JTRS, padding, strides)
    padv = np.finfo(np.float32).min if op == "max" else 0.0
    I2 = _slicable(np.asarray(I, dtype=np.float32), padv)
    O = np.empty(KMPQ + (N,), dtype=np.float32)
    for (k, m, p, q), idx in _pool_windows(C, DHW, JTRS, padding, strides, KMPQ):
        if op == "max":
            O[k, m, p, q, :] = np.max(I2[idx, :], axis=0)
        elif op == "avg":
            O[k, m, p, q, :] = np.mean(I2[idx, :].astype(np.float64), axis=0)
        elif op == "l2":
            O[k, m, p, q, :] = np.sqrt(np.sum(I2[idx, :].astype(np.float64) ** 2, axis=0))
        else:
            raise ValueError(op)
    return O


def ref_pool_fprop_pixels(I, op, JTRS, windows, padding=(0, 0, 0, 0), strides=None):
    """ref_pool_fprop restricted to a list of (k,m,p,q) outputs; returns (len, N)."""
    C, DHW, N, strides, KMPQ = _pool_setup(I.shape, JTRS, padding, strides)
    padv = np.finfo(np.float32).min if op == "max" else 0.0
    I2 = I.reshape(-1, N)
    imax = I2.shape[0]
    out = np.empty((len(windows), N), dtype=np.float32)
    for i, (k, m, p, q) in enumerate(windows):
        idx = pool_pixel_indices(C, DHW, JTRS, k * strides[0] - padding[0],
                                 m * strides[1] - padding[1], p * strides[2] - padding[2],
                                 q * strides[3] - padding[3])
        vals = np.full((idx.size, N), padv, dtype=np.float32)
        ok = idx < imax
        vals[ok] = I2[idx[ok]]
        out[i] = np.max(vals, axis=0) if op == "max" else np.mean(vals.astype(np.float64), axis=0)
    return out


def ref_pool_bprop(I, E, op, JTRS, padding=(0, 0, 0, 0), strides=None):
    """max: gradI[first argmax of the window] += E (benchmarks/pool_test.py:125-140;
    first-maximum tie rule kernels/sass/hpool_max.sass:264-282).
    avg: the adjoint of the avg fprop, gradI[slot] += E / (J*T*R*S) for in-bounds
    slots (the reference defines no avg bprop, pool_test.py:142)."""
    C, DHW, N, strides, KMPQ = _pool_setup(I.shape, JTRS, padding, strides)
    padv = np.finfo(np.float32).min if op == "max" else 0.0
    I2 = _slicable(np.asarray(I, dtype=np.float32), padv)
    E = np.asarray(E, dtype=np.float64)
    B = np.zeros(I2.shape, dtype=np.float64)
    ncols = np.arange(N)
    jrst = float(np.prod(JTRS))
    for (k, m, p, q), idx in _pool_windows(C, DHW, JTRS, padding, strides, KMPQ):
        if op == "max":
            b_idx = np.argmax(I2[idx, :], axis=0)
            np.add.at(B, (idx[b_idx], ncols), E[k, m, p, q, :])
        elif op == "avg":
            B[idx, :] += E[k, m, p, q, :][None, :] / jrst
        else:
            raise ValueError(op)
    return B[:-1].reshape(I.shape).astype(np.float32)


# --------------------------------------------------------------------------
# elementwise / reduction expressions
# --------------------------------------------------------------------------

def _f32(x):
    return np.asarray(x, dtype=np.float32)


_BINARY = {
    "add": lambda a, b: a + b,
    "sub": lambda a, b: a - b,
    "mul": lambda a, b: a * b,
    "div": lambda a, b: a / b,
    "pow": lambda a, b: np.power(a, b),
    "eq": lambda a, b: (a == b),
    "ne": lambda a, b: (a != b),
    "lt": lambda a, b: (a < b),
    "le": lambda a, b: (a <= b),
    "gt": lambda a, b: (a > b),
    "ge": lambda a, b: (a >= b),
    "minimum": lambda a, b: np.fmin(a, b),
    "maximum": lambda a, b: np.fmax(a, b),
}

_UNARY = {
    "neg": lambda a: -a,
    "abs": lambda a: np.abs(a),
    "sgn": lambda a: np.copysign(np.float32(1.0), a),
    "sqrt": lambda a: np.sqrt(a),
    "sqr": lambda a: a * a,
    "exp": lambda a: np.exp(a),
    "exp2": lambda a: np.exp2(a),
    "log": lambda a: np.log(a),
    "log2": lambda a: np.log2(a),
    "sig": lambda a: 1.0 / (1.0 + np.exp(-a)),
    "sig2": lambda a: 1.0 / (1.0 + np.exp2(-a)),
    "tanh": lambda a: np.tanh(a),
    "tanh2": lambda a: (np.exp2(2.0 * a) - 1.0) / (np.exp2(2.0 * a) + 1.0),
    "finite": lambda a: np.isfinite(a),
}


def ref_ew(stack, out_shape=None, rand=None, compute_dtype=np.float32):
    """Evaluate a postfix expression stack (numpy arrays, python scalars and op
    dicts) the way the generated kernels do: operands converted to fp32, every op
    in fp32 registers (op table nervanagpu/float_ew.py:464-495, reductions
    :497-533, composites nervanagpu/nervanagpu.py:1164-1224).  Reductions keep
    the reduced axis with length 1 and accumulate in float64.  Returns the fp32
    pre-rounding value (argmax/argmin as float32 indices).  `rand` supplies the
    uniform values for a `rand` op (callable shape->array)."""
    st = []
    cd = compute_dtype
    with np.errstate(all="ignore"):
        for item in stack:
            if isinstance(item, dict):
                op = item["op"]
                if op in _BINARY:
                    b = st.pop()
                    a = st.pop()
                    st.append(np.asarray(_BINARY[op](a, b)).astype(cd))
                elif op in _UNARY:
                    a = st.pop()
                    st.append(np.asarray(_UNARY[op](a)).astype(cd))
                elif op in ("sum", "max", "min", "argmax", "argmin"):
                    a = np.asarray(st.pop())
                    ax = item["axis"]
                    if op == "sum":
                        r = np.sum(a.astype(np.float64), axis=ax, keepdims=True)
                    elif op == "max":
                        r = np.max(a, axis=ax, keepdims=True)
                    elif op == "min":
                        r = np.min(a, axis=ax, keepdims=True)
                    elif op == "argmax":
                        r = np.expand_dims(np.argmax(a, axis=ax), ax)
                    else:
                        r = np.expand_dims(np.argmin(a, axis=ax), ax)
                    st.append(np.asarray(r).astype(cd))
                elif op == "rand":
                    st.append(np.asarray(rand(out_shape)).astype(cd))
                elif op == "onehot":
                    idx = np.asarray(item["idx"]).reshape(-1)
                    ax = item["axis"]
                    rows, cols = out_shape
                    if ax == 0:
                        # hot row index per column
                        r = (np.arange(rows)[:, None] == idx[None, :])
                    else:
                        r = (np.arange(cols)[None, :] == idx[:, None])
                    st.append(r.astype(cd))
                else:
                    raise ValueError("bad op %s" % op)
            elif isinstance(item, (int, float)):
                st.append(cd(item))
            else:
                st.append(np.asarray(item).astype(cd))
    assert len(st) == 1
    res = np.asarray(st[0], dtype=np.float32)
    if out_shape is not None:
        res = np.broadcast_to(res, out_shape)
    return res


def ref_batchnorm_rows(A, eps):
    """Closed form of A[:] = (A - mean(A,1)) / sqrt(var(A,1) + eps) with the
    population variance (nervanagpu/nervanagpu.py:1191-1208, README.md:113) in
    float64; fp32 pre-rounding value."""
    a = np.asarray(A, dtype=np.float64)
    mu = a.mean(axis=1, keepdims=True)
    var = ((a - mu) ** 2).mean(axis=1, keepdims=True)
    return ((a - mu) / np.sqrt(var + eps)).astype(np.float32)


def ref_transpose(a):
    """2-D transpose copy (nervanagpu/float_ew.py:1336-1365)."""
    return np.ascontiguousarray(np.asarray(a).T)


def ref_dimshuffle(F):
    """out[k,t,r,s,c] = in[c,t,r,s,k] (nervanagpu/float_ew.py:1377-1419)."""
    return np.ascontiguousarray(np.transpose(np.asarray(F), (4, 1, 2, 3, 0)))


def ref_compensated_sum(s, c, a, cmp_scale=1.0, add_scale=1.0, dtype=np.float16,
                        rounding=0, r=None):
    """Kahan-compensated accumulate in low precision
    (nervanagpu/float_ew.py:1453-1475).  Returns (new_sum, new_cmp) in `dtype`."""
    s32, c32, a32 = _f32(np.asarray(s, dtype=dtype)), _f32(np.asarray(c, dtype=dtype)), _f32(np.asarray(a, dtype=dtype))
    y32 = (a32 * np.float32(add_scale) - c32 * np.float32(cmp_scale)).astype(np.float32)
    rnd_sum = (s32 + y32).astype(np.float32)
    t = round_store(rnd_sum, dtype, rounding, r)
    t32 = _f32(t)
    rnd_cmp = ((t32 - s32).astype(np.float32) - y32).astype(np.float32)
    cc = round_store(rnd_cmp, dtype, 0)
    return t, cc
