"""numpy restatement of the CudaDnnDLL primitives and the C# attention layers.

TEST INFRASTRUCTURE ONLY (parity checker).  Every function names the reference
routine whose index arithmetic / call order it follows; paths are relative to
the reference tree.  ``dtype`` selects the arithmetic type (float32 mirrors the
reference's ``Kernel<float>``, float64 gives a tighter mathematical reference).

Pins (tests/test_oracle_layers.py): the inline vectors of
MyCaffe.test/TestCudaDnn.cs (gemm, gemv, mask, mask_batch, channel_copy), the
``gpt-pico-csa*`` golden tensors held by the reference test data (q after
transpose, softmax probabilities, y), scipy/torch library routines (softmax,
scaled_dot_product_attention, BLAS dgemm on column-major views for gemm2,
embedding, linear, multi_head_attention_forward for the whole multi-head layer
with causal / key-padding / per-batch masks) and closed forms (RoPE as a complex
rotation, the cos/sin tables).  Every function of this file has such a check.
"""
import numpy as np

MASKED = -1e29  # CausalSelfAttentionLayer.cs:60, attn.cu:307,324


# ----------------------------------------------------------------------------
# BLAS-like primitives
# ----------------------------------------------------------------------------

def gemm(transA, transB, m, n, k, alpha, A, B, beta, C=None, dtype=np.float32):
    """Row-major C[m,n] = alpha*op(A)*op(B) + beta*C.

    CudaDnnDLL/Cuda Files/math.cu:1481-1505: A is stored (m,k) or, transposed,
    (k,m); B is stored (k,n) or, transposed, (n,k).
    """
    A = np.asarray(A, dtype).reshape(-1)
    B = np.asarray(B, dtype).reshape(-1)
    a = A[:m * k].reshape((k, m)).T if transA else A[:m * k].reshape((m, k))
    b = B[:k * n].reshape((n, k)).T if transB else B[:k * n].reshape((k, n))
    out = dtype(alpha) * (a @ b)
    if beta != 0:
        out = out + dtype(beta) * np.asarray(C, dtype).reshape(-1)[:m * n].reshape(m, n)
    return out.astype(dtype)


def gemv(transA, m, n, alpha, A, x, beta, y=None, dtype=np.float32):
    """A is row-major (m,n); y = alpha*A*x + beta*y, or with transA y = alpha*A^T*x.

    math.cu:2101-2121 (cublasSgemv with the operation flag inverted because the
    row-major matrix is a column-major (n,m) matrix).
    """
    a = np.asarray(A, dtype).reshape(-1)[:m * n].reshape(m, n)
    xv = np.asarray(x, dtype).reshape(-1)
    out = dtype(alpha) * ((a.T @ xv[:m]) if transA else (a @ xv[:n]))
    if beta != 0:
        out = out + dtype(beta) * np.asarray(y, dtype).reshape(-1)[:out.size]
    return out.astype(dtype)


def gemm2_colmajor(transA, transB, m, n, k, alpha, A, B, beta, C, lda, ldb, ldc,
                   strideA=0, strideB=0, strideC=0, batch=1, dtype=np.float32):
    """cublasSgemmStridedBatched semantics on flat buffers (math.cu:1750-1788).

    Column-major: op(A) is (m,k), op(B) is (k,n), C is (m,n) with leading
    dimensions lda/ldb/ldc.  Returns the updated flat C.
    """
    A = np.asarray(A, dtype).reshape(-1)
    B = np.asarray(B, dtype).reshape(-1)
    C = np.array(C, dtype, copy=True).reshape(-1)

    def colview(buf, off, rows, cols, ld):
        idx = off + np.arange(rows)[:, None] + ld * np.arange(cols)[None, :]
        return idx

    for b in range(batch):
        ar, ac = (k, m) if transA else (m, k)
        br, bc = (n, k) if transB else (k, n)
        a = A[colview(A, b * strideA, ar, ac, lda)]
        bb = B[colview(B, b * strideB, br, bc, ldb)]
        a = a.T if transA else a
        bb = bb.T if transB else bb
        ci = colview(C, b * strideC, m, n, ldc)
        C[ci] = dtype(alpha) * (a @ bb) + (dtype(beta) * C[ci] if beta != 0 else 0)
    return C


def matmul(outer, m, n, k, A, B, scale=1.0, transA=False, transB=False, dtype=np.float32):
    """Row-major batched C[outer,m,n] = scale * op(A) @ op(B).

    MyCaffe/common/CudaDnn.cs:7513-7524: implemented by the host as a
    column-major gemm2 with the operands swapped.
    """
    lda = m if transA else k
    ldb = k if transB else n
    C = np.zeros(outer * m * n, dtype)
    C = gemm2_colmajor(transB, transA, n, m, k, scale, B, A, 0.0, C, ldb, lda, n,
                       k * n, m * k, m * n, outer, dtype=dtype)
    return C.reshape(outer, m, n)


def mask(n, mask_dim, search, replace, x, msk, dtype=np.float32):
    """y[i] = replace if mask[i % mask_dim] == search else x[i] (math.cu:2995-3002)."""
    x = np.asarray(x, dtype).reshape(-1)[:n]
    msk = np.asarray(msk, dtype).reshape(-1)
    idx = np.arange(n) % mask_dim
    return np.where(msk[idx] == dtype(search), dtype(replace), x).astype(dtype)


def mask_batch(n, batch, mask_dim, search, replace, x, msk, dtype=np.float32):
    """math.cu:3046-3056: mask index = i % (mask_dim/batch) + (i / (n/batch)) * (mask_dim/batch)."""
    x = np.asarray(x, dtype).reshape(-1)[:n]
    msk = np.asarray(msk, dtype).reshape(-1)
    md1 = mask_dim // batch
    dd1 = n // batch
    i = np.arange(n)
    idx = i % md1 + (i // dd1) * md1
    return np.where(msk[idx] == dtype(search), dtype(replace), x).astype(dtype)


def channel_copy_fwd(count, num, channels, blocks, inner, offset, x, dtype=np.float32):
    """Y[n,c,:] = X[n,c,offset,:] for X of shape (num, channels, blocks, inner) (math.cu:7510-7523)."""
    x = np.asarray(x, dtype).reshape(-1)
    i = np.arange(count)
    nn = i // (channels * inner)
    c = (i % (channels * inner)) // inner
    b = i % inner
    src = nn * channels * blocks * inner + c * blocks * inner + offset * inner + b
    return x[src].astype(dtype)


def channel_copy_bwd(count, num, channels, blocks, inner, offset, x, y, dtype=np.float32):
    """X[n,c,offset,:] = Y[n,c,:] (math.cu:7525-7539); returns the updated flat X."""
    x = np.array(x, dtype, copy=True).reshape(-1)
    y = np.asarray(y, dtype).reshape(-1)
    i = np.arange(count)
    nn = i // (channels * inner)
    c = (i % (channels * inner)) // inner
    b = i % inner
    dst = nn * channels * blocks * inner + c * blocks * inner + offset * inner + b
    x[dst] = y[:count]
    return x


def transpose(x, x_strides, y_strides, mapping, dtype=np.float32):
    """Generic permute of math.cu:4545-4571.

    ``x_strides[i]``/``y_strides[i]`` are the element strides of axis i of the
    source / destination (what the host passes as the "counts" blobs) and
    ``mapping[i]`` is the source axis that becomes destination axis i.
    """
    x = np.asarray(x, dtype).reshape(-1)
    n = x.size
    y = np.zeros(n, dtype)
    idx = np.arange(n)
    rem = idx.copy()
    from_inds = []
    for s in x_strides:
        from_inds.append(rem // int(s))
        rem = rem % int(s)
    to = np.zeros(n, np.int64)
    for i, s in enumerate(y_strides):
        to += from_inds[int(mapping[i])] * int(s)
    y[to] = x[idx]
    return y


def transpose_hw(n, c, h, w, x, dtype=np.float32):
    """(n,c,h,w) -> (n,c,w,h) (math.cu:4618-4654)."""
    return np.asarray(x, dtype).reshape(n * c, h, w).transpose(0, 2, 1).copy().reshape(-1)


def softmax_lastaxis(x, dtype=np.float32):
    """Max-subtracted softmax over the last axis (cudnnSoftmaxForward ACCURATE,
    memory.cu:2266-2288; CAFFE-engine chain SoftmaxLayer.cs:230-273)."""
    x = np.asarray(x, dtype)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return (e / e.sum(axis=-1, keepdims=True)).astype(dtype)


def softmax_backward(y, dy, axis=-1, log=False, dtype=np.float32):
    """Gradient with respect to the softmax input along ``axis`` from the output y and its gradient dy
    (cudnnSoftmaxBackward as SoftmaxLayer.cs:359-367 calls it): (dy - sum(dy * y)) * y, or, for the log form,
    dy - exp(y) * sum(dy)."""
    y, dy = np.asarray(y, dtype), np.asarray(dy, dtype)
    if log:
        return (dy - np.exp(y) * dy.sum(axis=axis, keepdims=True)).astype(dtype)
    return ((dy - (dy * y).sum(axis=axis, keepdims=True)) * y).astype(dtype)


def channel_max(x, num, channels, spatial, return_idx=False, across=True, dtype=np.float32):
    """channel_max kernels (math.cu:6697-6778).  across: y[n, s] = max_c x[n, c, s] (or the first index of it);
    within a channel the kernel walks num * spatial rows of `spatial` values: y[i] = max_j x[i * spatial + j]."""
    x = np.asarray(x, dtype).reshape(-1)
    if across:
        v = x[:num * channels * spatial].reshape(num, channels, spatial)
        return (np.argmax(v, axis=1).astype(dtype) if return_idx else v.max(axis=1)).reshape(-1)
    v = x[:num * spatial * spatial].reshape(num * spatial, spatial)
    return np.argmax(v, axis=1).astype(dtype) if return_idx else v.max(axis=1)


def channel_sub(a, x, num, channels, spatial, dtype=np.float32):
    """channel_sub_kernel (math.cu:6908-6916): y[n, c, s] = a[n, c, s] - x[n, s]."""
    return (np.asarray(a, dtype).reshape(num, channels, spatial) - np.asarray(x, dtype).reshape(num, 1, spatial)).reshape(-1)


def channel_div(y, x, num, channels, spatial, dtype=np.float32):
    """channel_div_kernel (math.cu:7160-7168): y[n, c, s] /= x[n, s]."""
    return (np.asarray(y, dtype).reshape(num, channels, spatial) / np.asarray(x, dtype).reshape(num, 1, spatial)).reshape(-1)


def channel_dot(x, a, num, channels, spatial, dtype=np.float32):
    """channel_dot_kernel (math.cu:7335-7351): y[n, s] = sum_c x[n, c, s] a[n, c, s], accumulated in double."""
    v = np.asarray(x, np.float64).reshape(num, channels, spatial) * np.asarray(a, np.float64).reshape(num, channels, spatial)
    return v.sum(axis=1).astype(dtype).reshape(-1)


def softmax_caffe_chain(x, axis, log=False, dtype=np.float32):
    """SoftmaxLayer.forward_cuda (SoftmaxLayer.cs:230-273) step by step on the primitives above."""
    x = np.asarray(x, dtype)
    axis %= x.ndim
    num, ch, sp = int(np.prod(x.shape[:axis], dtype=np.int64)), x.shape[axis], int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    top = x.reshape(-1).copy()
    c = channel_max(top, num, ch, sp, dtype=dtype)
    top = channel_sub(top, c, num, ch, sp, dtype)
    top = np.exp(top).astype(dtype)
    ssum = top.reshape(num, ch, sp).sum(axis=1).reshape(-1)
    if log:
        logz = c + np.log(ssum).astype(dtype)
        return channel_sub(x.reshape(-1), logz, num, ch, sp, dtype).reshape(x.shape)
    return channel_div(top, ssum, num, ch, sp, dtype).reshape(x.shape)


def silu(x, dtype=np.float32):
    """x * sigmoid(x) (math.cu:11699-11707)."""
    x = np.asarray(x, dtype)
    return (x * (dtype(1) / (dtype(1) + np.exp(-x)))).astype(dtype)


def embed_fwd(ids, weight, dtype=np.float32):
    """top[n,:] = weight[(int)ids[n],:] (math.cu:9314-9330)."""
    w = np.asarray(weight, dtype)
    return w[np.asarray(ids).astype(np.int64).reshape(-1)]


def rmsnorm_layer(x, weight=None, eps=1e-5, dtype=np.float32):
    """RMSNormLayer.cs:156-180: x / sqrt(mean(x^2, last axis) + eps) [* weight].

    channel_mean accumulates in double in the reference kernel
    (math.cu:6816-6830) and casts the mean to T.
    """
    x = np.asarray(x, dtype)
    ms = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True).astype(dtype)
    inv = dtype(1) / np.sqrt(ms + dtype(eps))
    out = x * inv
    if weight is not None:
        out = out * np.asarray(weight, dtype)
    return out.astype(dtype)


def rmsnorm_layer_backward(x, weight, dy, eps=1e-5, dtype=np.float32):
    """Gradients of ``rmsnorm_layer`` with weights as RMSNormLayer.cs:189-232 computes them, step by step: returns
    (dx, dw).  dw is what the layer's channel_sum call leaves in the weight gradient: the call sums over the axis
    before the last one for every leading index and the gradient blob holds one row, so it is the first leading
    entry's sum (for an input with one leading entry, the full gradient)."""
    x, dy, w = np.asarray(x, dtype), np.asarray(dy, dtype), np.asarray(weight, dtype)
    inner = x.shape[-1]
    x2 = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True).astype(dtype)
    x4 = np.sqrt(x2 + dtype(eps))
    x5 = dtype(1) / x4
    out = x * x5
    lead = x.reshape((-1,) + x.shape[-2:])                       # (outer, channels, inner)
    dw = (dy * out).reshape(lead.shape)[0].sum(axis=0)
    dout = dy * w
    dx_a = dout * x5
    dx5 = (dout * x).sum(axis=-1, keepdims=True)
    dx4 = dx5 * (dtype(-1) / (x4 * x4))
    dx2 = dx4 * (dtype(1) / (dtype(2) * x4))
    dx1 = np.broadcast_to(dx2, x.shape) / dtype(inner)
    return (dx_a + dtype(2) * x * dx1).astype(dtype), dw.astype(dtype)


# ----------------------------------------------------------------------------
# RoPE, CudaDnnDLL form
# ----------------------------------------------------------------------------

def rope_tables(seq_len, hs, theta=10000.0, base_double=False):
    """cos/sin tables [seq_len, hs/2] as RopeDataGpu<float>::Initialize builds
    them on the host (rope.cu:535-553): freq_j = 1/powf(theta, 2j/hs) in fp32,
    angle = freq_j * pos in fp32, cosf/sinf.  ``base_double``: the T = double
    instance of the same lines - the exponent, the reciprocal and the angle are
    held in double, powf / cosf / sinf still take and return floats."""
    if base_double:
        j = np.arange(0, hs, 2, dtype=np.float64)
        power = np.power(np.float32(theta), (j / np.float64(hs)).astype(np.float32), dtype=np.float32).astype(np.float64)
        freq = 1.0 / power
        ang = (freq[None, :] * np.arange(seq_len, dtype=np.float64)[:, None]).astype(np.float32)
        return np.cos(ang).astype(np.float32).astype(np.float64), np.sin(ang).astype(np.float32).astype(np.float64)
    j = np.arange(0, hs, 2, dtype=np.float32)
    power = (j / np.float32(hs)).astype(np.float32)
    freq = (np.float32(1.0) / np.power(np.float32(theta), power, dtype=np.float32)).astype(np.float32)
    pos = np.arange(seq_len, dtype=np.float32)[:, None]
    ang = (freq[None, :] * pos).astype(np.float32)
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def rope_forward(x, seq_len, heads, hs, theta=10000.0, freq_offset=-1, dtype=np.float32, base_double=False):
    """RopeDataGpu<T>::Forward (rope.cu:725-825).

    x is flat with an even count; consecutive (even, odd) elements form a pair.
    Pair i uses table entry ((i % (seq_len*heads*hs/2)) / (heads*hs/2)) * hs/2
    + i % (hs/2), shifted by freq_offset when freq_offset > 0.
    """
    x = np.asarray(x, dtype).reshape(-1)
    half = hs // 2
    full = half * heads
    cos, sin = rope_tables(seq_len, hs, theta, base_double)
    cos = cos.reshape(-1).astype(dtype)
    sin = sin.reshape(-1).astype(dtype)
    off = freq_offset if freq_offset > 0 else 0
    i = np.arange(x.size // 2)
    base = i % (seq_len * full)
    t = (base // full) * half + base % half + off
    re, im = x[0::2], x[1::2]
    y = np.empty_like(x)
    y[0::2] = re * cos[t] - im * sin[t]
    y[1::2] = re * sin[t] + im * cos[t]
    return y


# ----------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------

def attn_forward(q, k, v, mask_data=None, batch_mask=False, dtype=np.float32):
    """attnHandle<T>::Forward (attn.cu:518-602).

    q, k, v: (B,H,T,hs).  mask (1,1,T,T) when batch_mask is False (zero entries
    are filled with -1e29), (B,T) key mask when True.  Returns (y, probs).
    """
    q = np.asarray(q, dtype)
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    B, H, T, hs = q.shape
    scale = dtype(1.0 / np.sqrt(float(hs)))
    att = (q @ k.transpose(0, 1, 3, 2)) * scale
    if mask_data is not None:
        m = np.asarray(mask_data, dtype)
        if batch_mask:
            att = mask_batch(att.size, B, m.size, 0.0, MASKED, att, m, dtype).reshape(att.shape)
        else:
            att = mask(att.size, m.size, 0.0, MASKED, att, m, dtype).reshape(att.shape)
    p = softmax_lastaxis(att, dtype)
    return (p @ v).astype(dtype), p


def inner_product(x, w, b=None, dtype=np.float32):
    """InnerProductLayer.forward (InnerProductLayer.cs:372-417): y = x W^T [+ 1 b],
    W stored (num_output, K)."""
    x = np.asarray(x, dtype)
    y = x @ np.asarray(w, dtype).T
    if b is not None:
        y = y + np.asarray(b, dtype)
    return y.astype(dtype)


def causal_mask(T, dtype=np.float32):
    """fillMask (CausalSelfAttentionLayer.cs:276-291): ones on and below the diagonal."""
    return np.tril(np.ones((T, T), dtype))


def causal_self_attention(x, w_attn, b_attn, w_proj, b_proj, heads, rope=None, dtype=np.float32):
    """CausalSelfAttentionLayer.forward (CausalSelfAttentionLayer.cs:526-628).

    x (B,T,C); fused QKV InnerProduct (3C,C); q,k,v are consecutive thirds of
    the fused output; heads split as (B,T,H,hs)->(B,H,T,hs); causal mask;
    softmax; @v; merge heads; output projection.  ``rope`` = (seq_len, theta)
    applies rope_forward to q and k before the head transpose.
    Returns dict with intermediates.
    """
    x = np.asarray(x, dtype)
    B, T, C = x.shape
    hs = C // heads
    qkv = inner_product(x, w_attn, b_attn, dtype)
    q, k, v = qkv[..., :C], qkv[..., C:2 * C], qkv[..., 2 * C:]
    if rope is not None:
        q = rope_forward(q, rope[0], heads, hs, rope[1], dtype=dtype).reshape(B, T, C)
        k = rope_forward(k, rope[0], heads, hs, rope[1], dtype=dtype).reshape(B, T, C)
    qt = q.reshape(B, T, heads, hs).transpose(0, 2, 1, 3)
    kt = k.reshape(B, T, heads, hs).transpose(0, 2, 1, 3)
    vt = v.reshape(B, T, heads, hs).transpose(0, 2, 1, 3)
    work, att = attn_forward(qt, kt, vt, causal_mask(T, dtype), False, dtype)
    ymerged = work.transpose(0, 2, 1, 3).reshape(B, T, C)
    y = inner_product(ymerged, w_proj, b_proj, dtype)
    return {"qt": qt, "kt": kt, "vt": vt, "att": att, "work": work, "y": y}


def multihead_attention(xq, xk, xv, wq, bq, wk, bk, wv, bv, wo, bo, heads, mask_data=None,
                        mask_kind="none", rope=None, position=-1, dtype=np.float32):
    """MultiheadAttentionLayer.forward without KV cache (MultiheadAttentionLayer.cs:643-811).

    mask_kind: "none", "causal" ((1,1,T,T) tril), "key" ((B,T_k) key padding,
    broadcast over heads and query rows) or "full" ((B,T_q,T_k), broadcast over
    heads): the last two go through mask_batch.  Cross attention may use
    T_q != T_k here (the reference layer assumes equal lengths; the closed form
    is the same).
    """
    xq = np.asarray(xq, dtype)
    xk = np.asarray(xk, dtype)
    xv = np.asarray(xv, dtype)
    B, Tq, C = xq.shape
    Tk = xk.shape[1]
    hs = C // heads
    q = inner_product(xq, wq, bq, dtype)
    k = inner_product(xk, wk, bk, dtype)
    v = inner_product(xv, wv, bv, dtype)
    if rope is not None:
        off = position * hs // 2 if position > 0 else -1
        q = rope_forward(q, rope[0], heads, hs, rope[1], off, dtype).reshape(B, Tq, C)
        k = rope_forward(k, rope[0], heads, hs, rope[1], off, dtype).reshape(B, Tk, C)
    qt = q.reshape(B, Tq, heads, hs).transpose(0, 2, 1, 3)
    kt = k.reshape(B, Tk, heads, hs).transpose(0, 2, 1, 3)
    vt = v.reshape(B, Tk, heads, hs).transpose(0, 2, 1, 3)
    scale = dtype(1.0 / np.sqrt(float(hs)))
    att = (qt @ kt.transpose(0, 1, 3, 2)) * scale
    if mask_kind == "causal":
        m = np.asarray(mask_data, dtype)
        att = mask(att.size, m.size, 0.0, MASKED, att, m, dtype).reshape(att.shape)
    elif mask_kind in ("key", "full"):
        m = np.asarray(mask_data, dtype)
        att = mask_batch(att.size, B, m.size, 0.0, MASKED, att, m, dtype).reshape(att.shape)
    p = softmax_lastaxis(att, dtype)
    work = p @ vt
    y = inner_product(work.transpose(0, 2, 1, 3).reshape(B, Tq, C), wo, bo, dtype)
    return {"qt": qt, "kt": kt, "vt": vt, "att": p, "work": work, "y": y}


def kv_cache_attention(q, kcache, vcache, dtype=np.float32):
    """KV-cache branch of MultiheadAttentionLayer (MultiheadAttentionLayer.cs:713-730,
    759-777) and the per-head loop of llama2_cpu.cpp:306-341: one query per head,
    scores = q.k_t/sqrt(hs) over all cached t, softmax without a mask, sum_t p_t v_t.

    q (B,H,hs); kcache, vcache (B,H,L,hs).  Returns (B,H,hs).
    """
    q = np.asarray(q, dtype)
    kc = np.asarray(kcache, dtype)
    vc = np.asarray(vcache, dtype)
    hs = q.shape[-1]
    s = np.einsum("bhd,bhld->bhl", q, kc) / dtype(np.sqrt(float(hs)))
    p = softmax_lastaxis(s, dtype)
    return np.einsum("bhl,bhld->bhd", p, vc).astype(dtype)


# ----------------------------------------------------------------------------
# LayerNorm handle, GELU / SiLU, gradients
# ----------------------------------------------------------------------------

def layernorm_forward(x, inner, eps=1e-10, dtype=np.float32):
    """LayerNormData::Forward (CudaDnnDLL/Cuda Files/layernorm.cu:219-262): per row of ``inner`` values
    mean -> xmu = x - mean -> var = mean(xmu^2) -> stdev = sqrt(var + eps) -> y = xmu / stdev.  No affine part.
    Returns (y, stdev[rows])."""
    x = np.asarray(x, dtype)
    r = x.reshape(-1, inner)
    mu = (r.astype(np.float64).sum(1) / inner).astype(dtype)          # channel_mean accumulates in double (math.cu:6817-6831)
    xmu = r - mu[:, None]
    var = ((xmu * xmu).astype(np.float64).sum(1) / inner).astype(dtype)
    stdev = np.sqrt(var + dtype(eps)).astype(dtype)
    return (xmu / stdev[:, None]).astype(dtype).reshape(x.shape), stdev


def layernorm_backward(y, dy, stdev, inner, eps=1e-10, backward_calls=1, dtype=np.float32):
    """LayerNormData::Backward (layernorm.cu:268-312): dx = (dy - (y * mean(y*dy) + mean(dy))) / stdev_full.

    stdev_full is the row-expanded stdev array of the forward pass; before the division the reference adds eps to
    its first ``rows`` flat entries (``add_scalar(outer*channels, eps, stdevfull)``, layernorm.cu:306), once per
    backward call and cumulatively until the next forward refills the array."""
    y = np.asarray(y, dtype)
    r = y.reshape(-1, inner)
    g = np.asarray(dy, dtype).reshape(-1, inner)
    rows = r.shape[0]
    m1 = ((r * g).astype(np.float64).sum(1) / inner).astype(dtype)
    m2 = (g.astype(np.float64).sum(1) / inner).astype(dtype)
    work = g - (r * m1[:, None] + m2[:, None])
    full = np.repeat(np.asarray(stdev, dtype), inner)
    for _ in range(backward_calls):
        full[:rows] = full[:rows] + dtype(eps)
    return (work / full.reshape(rows, inner)).astype(dtype).reshape(y.shape)


def gelu(x, bert, dtype=np.float32):
    """gelu_fwd_kernel / gelu_fwd_kernel_bert (math.cu:11348-11376).  The tanh form is evaluated in double on the
    T-typed input and constant and cast back; the erf form stays in T."""
    from scipy.special import erf
    x = np.asarray(x, dtype)
    if bert:
        k = np.float64(dtype(np.sqrt(2.0 / np.pi)))
        x3 = (x * x * x).astype(np.float64)
        xd = x.astype(np.float64)
        return (0.5 * xd * (1.0 + np.tanh(k * (xd + 0.044715 * x3)))).astype(dtype)
    return (x * (dtype(0.5) * (dtype(1.0) + erf(x / dtype(np.sqrt(2.0))).astype(dtype)))).astype(dtype)


def gelu_grad(x, dy, bert, dtype=np.float32):
    """gelu_bwd_kernel / gelu_bwd_kernel_bert (math.cu:11412-11448) with the reference's rounded constants."""
    from scipy.special import erf
    x = np.asarray(x, dtype)
    dy = np.asarray(dy, dtype)
    if bert:
        x3 = x * x * x
        t = dtype(0.797885) * (x + dtype(0.044715) * x3)
        vx = dtype(0.0535161) * x3 + dtype(0.398942) * x
        ch = np.cosh(t)
        grad = dtype(0.5) * np.tanh(t) + vx * (dtype(1.0) / (ch * ch)) + dtype(0.5)
    else:
        cdf = dtype(0.5) * (dtype(1.0) + erf(x / dtype(np.sqrt(2.0))).astype(dtype))
        pdf = dtype(1.0) / dtype(np.sqrt(2.0 * np.pi)) * np.exp(dtype(-0.5) * (x * x))
        grad = cdf + x * pdf
    return (dy * grad).astype(dtype)


def relu(x, slope=0.0, dtype=np.float32):
    """relu_fwd_kernel (math.cu:12038-12044)."""
    x = np.asarray(x, dtype)
    return np.where(x > 0, x, x * dtype(slope)).astype(dtype)


def relu_grad(y, dy, slope=0.0, dtype=np.float32):
    """relu_bwd_kernel (math.cu:12072-12078): the gate is read from the TOP data."""
    y = np.asarray(y, dtype)
    return (np.asarray(dy, dtype) * ((y > 0).astype(dtype) + (y <= 0).astype(dtype) * dtype(slope))).astype(dtype)


def silu_grad(x, dy, dtype=np.float32):
    """silu_bwd_kernel (math.cu:11740-11749): dy * s (1 + x (1 - s)), s = sigmoid(x)."""
    x = np.asarray(x, dtype)
    s = dtype(1.0) / (dtype(1.0) + np.exp(-x))
    return (np.asarray(dy, dtype) * (s * (dtype(1.0) + x * (dtype(1.0) - s)))).astype(dtype)


def rope_backward(dy, seq_len, heads, hs, theta=10000.0, dtype=np.float32):
    """RopeDataGpu::Backward (rope.cu:832-864, copy_computeRI_grad_kernel :754-770): the rotation by the opposite
    angle with the unshifted tables (the backward pass takes no frequency offset)."""
    dy = np.asarray(dy, dtype)
    flat = dy.reshape(-1)
    pairs = flat.size // 2
    half = hs // 2
    full = half * heads
    fcos, fsin = rope_tables(seq_len, hs, theta)
    p = np.arange(pairs)
    base = p % (seq_len * full)
    idx = (base // full) * half + base % half
    c = fcos.reshape(-1)[idx].astype(dtype)
    s = fsin.reshape(-1)[idx].astype(dtype)
    re, im = flat[0::2], flat[1::2]
    out = np.empty_like(flat)
    out[0::2] = re * c + im * s
    out[1::2] = -re * s + im * c
    return out.reshape(dy.shape)


def attn_backward(q, k, v, att, dy, dtype=np.float32):
    """attnHandle::Backward (attn.cu:608-661) without dropout, on the probabilities ``att`` saved by the forward pass:
    dV = att^T dY, dAtt = dY V^T (matmulgrad :380-397); softmax backward dS = att * (dAtt - rowsum(dAtt * att));
    dS *= 1/sqrt(hs); dQ = dS K, dK = dS^T Q.  Masked entries need no special case: their probability is exactly 0.
    All of q, k, v, dy (B,H,T,hs); returns (dq, dk, dv)."""
    q = np.asarray(q, dtype); k = np.asarray(k, dtype); v = np.asarray(v, dtype)
    att = np.asarray(att, dtype); dy = np.asarray(dy, dtype)
    scale = dtype(1.0 / np.sqrt(np.float64(q.shape[-1])))
    dv = np.swapaxes(att, -1, -2) @ dy
    datt = dy @ np.swapaxes(v, -1, -2)
    ds = att * (datt - (datt * att).sum(-1, keepdims=True))
    ds = ds * scale
    dq = ds @ k
    dk = np.swapaxes(ds, -1, -2) @ q
    return dq.astype(dtype), dk.astype(dtype), dv.astype(dtype)


def splitmix64(state):
    """One output of the SplitMix64 generator for each 64-bit ``state`` (Steele, Lea, Flood, "Fast splittable
    pseudorandom number generators", OOPSLA 2014; the increment is folded in: out = mix(state + golden))."""
    with np.errstate(over="ignore"):
        z = np.asarray(state, np.uint64) + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


ATTN_DROPOUT_CALL_STRIDE = 0xD1B54A32D192ED03   # the HIP handle adds this to the seed for every training-mode forward call


def attn_dropout_keep(seed, B, H, Tq, Tk, ratio, forward_calls=1):
    """Which probabilities survive attention dropout in the HIP library (the reference draws its mask from cuDNN's
    generator, attn.cu:261-276, whose stream cannot be restated; only the distribution and the forward / backward
    consistency carry over).  keep[b,h,i,j] = high 32 bits of splitmix64(seed' * golden + index) >= ratio * 2^32 with
    index = ((b*H + h)*Tq + i)*Tk + j and seed' = seed + forward_calls * ATTN_DROPOUT_CALL_STRIDE."""
    with np.errstate(over="ignore"):
        seed2 = np.uint64((int(seed) + forward_calls * ATTN_DROPOUT_CALL_STRIDE) & 0xFFFFFFFFFFFFFFFF)
        idx = np.arange(B * H * Tq * Tk, dtype=np.uint64)
        r = splitmix64(seed2 * np.uint64(0x9E3779B97F4A7C15) + idx) >> np.uint64(32)
    thr = min(int(float(np.float32(ratio)) * 4294967296.0), 4294967295)
    return (r >= np.uint64(thr)).reshape(B, H, Tq, Tk)


def attn_forward_dropout(q, k, v, keep, ratio, mask_data=None, batch_mask=False, dtype=np.float32):
    """attnHandle::Forward in training mode with a dropout ratio (attn.cu:518-602): dropout is applied in place to the
    softmax probabilities (survivors scaled by 1 / (1 - ratio)) before the product with V.  Returns (y, probabilities
    before dropout, probabilities after)."""
    _, p = attn_forward(q, k, v, mask_data, batch_mask, dtype)
    pd = (p * (np.asarray(keep, dtype) * dtype(1.0 / (1.0 - float(np.float32(ratio)))))).astype(dtype)
    return (pd @ np.asarray(v, dtype)).astype(dtype), p, pd


def attn_backward_dropout(q, k, v, att_dropped, keep, ratio, dy, dtype=np.float32):
    """attnHandle::Backward with dropout, step by step as the reference runs it (attn.cu:608-661).  ``att_dropped`` is
    what m_blobAttB holds after the forward pass: the probabilities with dropout applied IN PLACE (:578-583).
      dV = AttB^T dY, dAttB = dY V^T                       (matmulgrad, :632-633)
      dAttB *= keep / (1 - ratio)                          (apply_dropout_bwd, :637-640)
      dAttA = AttB * (dAttB - rowsum(dAttB * AttB))        (softmax_bwd with y = the dropped AttB, :643-644)
      dQ = dAttA K / sqrt(hs), dK = dAttA^T Q / sqrt(hs)   (:647-652)
    Because the softmax backward reads the dropped probabilities, a dropped entry gets no gradient at all and a kept one
    carries 1 / (1 - ratio)^2; this is the reference's result, not the derivative of its forward pass."""
    q = np.asarray(q, dtype); k = np.asarray(k, dtype); v = np.asarray(v, dtype)
    attb = np.asarray(att_dropped, dtype); dy = np.asarray(dy, dtype)
    scale = dtype(1.0 / np.sqrt(np.float64(q.shape[-1])))
    dv = np.swapaxes(attb, -1, -2) @ dy
    datt = dy @ np.swapaxes(v, -1, -2)
    datt = datt * (np.asarray(keep, dtype) * dtype(1.0 / (1.0 - float(np.float32(ratio)))))
    ds = softmax_backward(attb, datt, axis=-1, log=False, dtype=dtype) * scale
    dq = ds @ k
    dk = np.swapaxes(ds, -1, -2) @ q
    return dq.astype(dtype), dk.astype(dtype), dv.astype(dtype)


def transformer_block_gpt(x, p, heads, activation="relu", eps=1e-10, dtype=np.float32):
    """TransformerBlockLayer.forward, CAUSAL_SELF_ATTENTION block type (TransformerBlockLayer.cs:810-902):
    xB = x + attn(ln1(x)); y = xB + proj(gelu(fc(ln2(xB)))).  ``p`` maps attn_weight, attn_bias, attn_proj_weight,
    attn_proj_bias, fc_weight, fc_bias, proj_weight, proj_bias; ``activation`` is "relu" (the layer's default,
    TransformerBlockLayer.cs:316), "gelu" or "gelu_bert".  Returns dict with the intermediates."""
    x = np.asarray(x, dtype)
    C = x.shape[-1]
    ln1, _ = layernorm_forward(x, C, eps, dtype)
    attn = causal_self_attention(ln1, p["attn_weight"], p["attn_bias"], p["attn_proj_weight"], p["attn_proj_bias"], heads,
                                 dtype=dtype)["y"]
    xb = (x + attn).astype(dtype)
    ln2, _ = layernorm_forward(xb, C, eps, dtype)
    fc = inner_product(ln2, p["fc_weight"], p["fc_bias"], dtype)
    act = relu(fc, 0.0, dtype) if activation == "relu" else gelu(fc, activation == "gelu_bert", dtype)
    mlp = inner_product(act, p["proj_weight"], p["proj_bias"], dtype)
    return {"ln1": ln1, "attn": attn, "xb": xb, "ln2": ln2, "fc": fc, "act": act, "mlp": mlp, "y": (xb + mlp).astype(dtype)}


def transformer_block_llama(x, p, heads, seq_len, theta=10000.0, eps=1e-5, dtype=np.float32):
    """TransformerBlockLayer.forward with enable_llama_style_head (TransformerBlockLayer.cs:810-902): RMSNorm, causal self
    attention with rotary q / k and no bias, xB = x + attn; y = xB + proj(silu(fc1(n)) * fc2(n)), n = RMSNorm(xB).
    ``p``: rms1_weight, rms2_weight, attn_weight, attn_proj_weight, fc_weight, fc2_weight, proj_weight."""
    x = np.asarray(x, dtype)
    n1 = rmsnorm_layer(x, p["rms1_weight"], eps, dtype)
    attn = causal_self_attention(n1, p["attn_weight"], None, p["attn_proj_weight"], None, heads, rope=(seq_len, theta), dtype=dtype)["y"]
    xb = (x + attn).astype(dtype)
    n2 = rmsnorm_layer(xb, p["rms2_weight"], eps, dtype)
    h = silu(inner_product(n2, p["fc_weight"], None, dtype), dtype) * inner_product(n2, p["fc2_weight"], None, dtype)
    return (xb + inner_product(h.astype(dtype), p["proj_weight"], None, dtype)).astype(dtype)
