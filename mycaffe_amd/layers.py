"""Host-side mirrors of the MyCaffe layers that call the attention hot path.

These follow the C# ``forward`` methods call for call (cited per class), so that a
forward pass here issues the same sequence of ``CudaDnn`` calls, with the same
argument packing, as the unchanged C# host would issue against the native library.
Dropout layers are the identity (inference, or training with ratio 0).  ``Backward`` is mirrored for the GPT block
(InnerProduct, Transpose, LayerNorm, activations, CausalSelfAttention with the fused attention handle, TransformerBlock).
"""
import math

import numpy as np

from .cudadnn import DIR, SOFTMAX_ALGORITHM, SOFTMAX_MODE


class Blob:
    """Shape + device handle, the part of MyCaffe/common/Blob.cs the layers use."""

    def __init__(self, cuda, shape=None, half=False):
        self.cuda = cuda
        self.half = half
        self.shape_ = []
        self.gpu_data = 0
        self._capacity = 0
        self._gpu_diff = 0
        self._diff_capacity = 0
        if shape is not None:
            self.Reshape(*shape)

    def Reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (list, tuple)):
            shape = tuple(shape[0])
        self.shape_ = [int(s) for s in shape]
        n = self.count()
        if n > self._capacity:
            if self.gpu_data:
                self.cuda.FreeMemory(self.gpu_data)
            self.gpu_data = self.cuda.AllocMemory(n, bHalfSize=self.half)
            self._capacity = n

    def ReshapeLike(self, other):
        self.Reshape(*other.shape_)

    def count(self, start=0, end=None):
        s = self.shape_[start:end]
        return int(np.prod(s)) if s else 1

    def shape(self, i):
        return self.shape_[i]

    num = property(lambda self: self.shape_[0])
    channels = property(lambda self: self.shape_[1] if len(self.shape_) > 1 else 1)
    height = property(lambda self: self.shape_[2] if len(self.shape_) > 2 else 1)
    width = property(lambda self: self.shape_[3] if len(self.shape_) > 3 else 1)
    num_axes = property(lambda self: len(self.shape_))
    mutable_gpu_data = property(lambda self: self.gpu_data)

    @property
    def gpu_diff(self):
        """Gradient buffer of the same size, allocated (zero filled) on first use."""
        n = self.count()
        if n > self._diff_capacity:
            if self._gpu_diff:
                self.cuda.FreeMemory(self._gpu_diff)
            self._gpu_diff = self.cuda.AllocMemory(n, bHalfSize=self.half)
            self._diff_capacity = n
        return self._gpu_diff

    mutable_gpu_diff = gpu_diff

    @property
    def mutable_cpu_diff(self):
        return self.cuda.GetMemoryFloat(self.gpu_diff, self.count()).reshape(self.shape_)

    @mutable_cpu_diff.setter
    def mutable_cpu_diff(self, values):
        self.cuda.SetMemory(self.gpu_diff, np.asarray(values, self.cuda.DTYPE).reshape(-1), nCount=self.count())

    @property
    def mutable_cpu_data(self):
        return self.cuda.GetMemoryFloat(self.gpu_data, self.count()).reshape(self.shape_)

    @mutable_cpu_data.setter
    def mutable_cpu_data(self, values):
        self.cuda.SetMemory(self.gpu_data, np.asarray(values, self.cuda.DTYPE).reshape(-1), nCount=self.count())

    def SetData(self, value):
        self.cuda.set(self.count(), self.gpu_data, float(value))

    def CopyFrom(self, src, bCopyDiff=False, bReshape=True):
        """Blob.cs CopyFrom(src, bCopyDiff, bReshape): copies the data, or with bCopyDiff the diff."""
        if bReshape:
            self.ReshapeLike(src)
        if bCopyDiff:
            self.cuda.copy(self.count(), src.gpu_diff, self.gpu_diff)
        else:
            self.cuda.copy(self.count(), src.gpu_data, self.gpu_data)

    def MatMul(self, blobA, blobB, bReshape=False, bTransA=False, bTransB=False, dfScale=1.0, bADiff=False, bBDiff=False,
               bCDiff=False, bAccumulate=False):
        """Blob.cs:4229-4269: batched row-major matmul over the two leading axes; the flags pick the diff side of each blob."""
        outer = blobA.count(0, 2)
        m = blobA.shape(3) if bTransA else blobA.shape(2)
        n = blobB.shape(2) if bTransB else blobB.shape(3)
        k = blobA.shape(2) if bTransA else blobA.shape(3)
        shape = [blobA.shape(0), blobB.shape(1), m, n]
        if bReshape:
            self.Reshape(*shape)
        elif self.shape_ != shape:
            raise ValueError("This (resulting) blob does not have the correct shape! Expected %s" % shape)
        hA = blobA.gpu_diff if bADiff else blobA.gpu_data
        hB = blobB.gpu_diff if bBDiff else blobB.gpu_data
        hC = self.gpu_diff if bCDiff else self.gpu_data
        self.cuda.matmul(outer, m, n, k, hA, hB, hC, dfScale, bTransA, bTransB, bAccumulate)

    def MatMulGrad(self, blobA, blobB, dfScale=1.0, bAccumulate=False):
        """Blob.cs:4304-4311: from this blob's diff, A.diff = dC B^T and B.diff = A^T dC."""
        if dfScale != 1.0:
            self.scale_diff(dfScale)
        blobA.MatMul(self, blobB, False, False, True, 1.0, True, False, True, bAccumulate)
        blobB.MatMul(blobA, self, False, True, False, 1.0, False, True, True, bAccumulate)

    def scale_data(self, df):
        self.cuda.scal(self.count(), df, self.gpu_data)

    def scale_diff(self, df):
        self.cuda.scal(self.count(), df, self.gpu_diff)

    def Dispose(self):
        if self.gpu_data:
            self.cuda.FreeMemory(self.gpu_data)
            self.gpu_data = 0
            self._capacity = 0
        if self._gpu_diff:
            self.cuda.FreeMemory(self._gpu_diff)
            self._gpu_diff = 0
            self._diff_capacity = 0


class InnerProductLayer:
    """MyCaffe/layers/InnerProductLayer.cs:372-417.  Weights are (num_output, K)."""

    def __init__(self, cuda, num_output, bias_term=True, axis=2, half=False, fused_bias=False):
        self.cuda, self.N, self.bias_term, self.axis, self.half = cuda, num_output, bias_term, axis, half
        # product and bias in one call (an id with no counterpart in the reference) instead of the two GEMM calls
        self.fused_bias = fused_bias
        self.blobs = []
        self.bias_multiplier = None

    def Setup(self, bottom, weight=None, bias=None):
        self.K = bottom.count(self.axis)
        w = Blob(self.cuda, (self.N, self.K), self.half)
        if weight is not None:
            w.mutable_cpu_data = weight
        self.blobs = [w]
        if self.bias_term:
            b = Blob(self.cuda, (self.N,), self.half)
            if bias is not None:
                b.mutable_cpu_data = bias
            self.blobs.append(b)

    def Forward(self, bottom, top):
        M = bottom.count(0, self.axis)
        top.Reshape(*(bottom.shape_[:self.axis] + [self.N]))
        hW = self.blobs[0].gpu_data
        if self.fused_bias:
            self.cuda.LinearForward(M, self.N, self.K, bottom.gpu_data, hW, self.blobs[1].gpu_data if self.bias_term else 0,
                                    top.gpu_data)
        elif M == 1 and not self.half:
            self.cuda.gemv(False, self.N, self.K, 1.0, hW, bottom.gpu_data, 0.0, top.gpu_data)
            if self.bias_term:
                self.cuda.axpy(self.N, 1.0, self.blobs[1].gpu_data, top.gpu_data)
        else:
            self.cuda.gemm(False, True, M, self.N, self.K, 1.0, bottom.gpu_data, hW, 0.0, top.gpu_data)
            if self.bias_term:
                if self.bias_multiplier is None or self.bias_multiplier.count() < M:
                    self.bias_multiplier = Blob(self.cuda, (M,), self.half)
                    self.bias_multiplier.SetData(1.0)
                self.cuda.gemm(False, False, M, self.N, 1, 1.0, self.bias_multiplier.gpu_data, self.blobs[1].gpu_data, 1.0,
                               top.gpu_data)


    def Backward(self, top, bottom):
        """InnerProductLayer.cs:429-494: weight gradient accumulates into the weight diff, bias gradient through gemv with
        the ones vector, data gradient = top diff x W."""
        M = bottom.count(0, self.axis)
        hTopDiff, hW = top.gpu_diff, self.blobs[0].gpu_data
        self.cuda.gemm(True, False, self.N, self.K, M, 1.0, hTopDiff, bottom.gpu_data, 1.0, self.blobs[0].gpu_diff)
        if self.bias_term:
            if self.bias_multiplier is None or self.bias_multiplier.count() < M:
                self.bias_multiplier = Blob(self.cuda, (M,), self.half)
                self.bias_multiplier.SetData(1.0)
            self.cuda.gemv(True, M, self.N, 1.0, hTopDiff, self.bias_multiplier.gpu_data, 1.0, self.blobs[1].gpu_diff)
        self.cuda.gemm(False, False, M, self.K, self.N, 1.0, hTopDiff, hW, 0.0, bottom.gpu_diff)


class TransposeLayer:
    """MyCaffe.layers.beta/layers.beta/TransposeLayer.cs:127-232."""

    def __init__(self, cuda, dim):
        self.cuda, self.dim = cuda, list(dim)
        self._key = None
        self._handles = []

    def _reshape(self, shape):
        """Reshape (TransposeLayer.cs:127-200): stride arrays of bottom and top, forward and backward axis maps."""
        key = (tuple(shape), tuple(self.dim))
        top_shape = [shape[d] for d in self.dim]
        if key != self._key:
            for h in self._handles:
                self.cuda.FreeMemory(h)
            n = len(shape)
            bc = [int(np.prod(shape[i + 1:])) for i in range(n)]
            tc = [int(np.prod(top_shape[i + 1:])) for i in range(n)]
            bmap = [0] * n
            for i, d in enumerate(self.dim):
                bmap[d] = i
            self.counts_b = self.cuda.AllocMemory(np.float32(bc))
            self.counts_t = self.cuda.AllocMemory(np.float32(tc))
            self.fmap = self.cuda.AllocMemory(np.float32(self.dim))
            self.bmap = self.cuda.AllocMemory(np.float32(bmap))
            self.buffer = self.cuda.AllocMemory(int(np.prod(shape)) * n)
            self._handles = [self.counts_b, self.counts_t, self.fmap, self.bmap, self.buffer]
            self._key = key
        return top_shape

    def Forward(self, bottom, top):
        if bottom.gpu_data == top.gpu_data:
            raise ValueError("The Transpose layer does not support in-place computation.")
        top.Reshape(*self._reshape(bottom.shape_))
        self.cuda.transpose(bottom.count(), bottom.gpu_data, top.gpu_data, self.counts_b, self.counts_t, self.fmap,
                            len(bottom.shape_), self.buffer)

    def Backward(self, top, bottom):
        """TransposeLayer.cs:223-232: reshape for this bottom, then the same kernel with the count arrays swapped and the
        inverse axis map."""
        self._reshape(bottom.shape_)
        self.cuda.transpose(bottom.count(), top.gpu_diff, bottom.gpu_diff, self.counts_t, self.counts_b, self.bmap,
                            len(bottom.shape_), self.buffer)


class SoftmaxLayer:
    """MyCaffe/layers/SoftmaxLayer.cs: the cuDNN engine (:172-181, 339-367) or, with ``engine="CAFFE"``, the chain of
    primitives of forward_cuda / backward_cuda (:230-330; ``algorithm="LOG"`` for the log-softmax variant)."""

    def __init__(self, cuda, axis=-1, engine="CUDNN", algorithm="ACCURATE"):
        self.cuda, self.axis, self.engine, self.algorithm = cuda, axis, engine, algorithm
        self.hCudnn = cuda.CreateCuDNN()
        self.hBottomDesc = cuda.CreateTensorDesc()
        self.hTopDesc = cuda.CreateTensorDesc()
        self.blobScale = None

    def _forward_caffe(self, bottom, top):
        """SoftmaxLayer.cs:230-273."""
        cuda = self.cuda
        axis = self.axis % bottom.num_axes
        nOuter, nCh, nInner = bottom.count(0, axis), bottom.shape(axis), bottom.count(axis + 1)
        top.ReshapeLike(bottom)
        if self.blobScale is None or self.blobScale.count() != nOuter * nInner or self.blobScale.half != bottom.half:
            self.blobScale = Blob(cuda, (nOuter, nInner), bottom.half)
        self._dims = (nOuter, nCh, nInner)
        hB, hT, hSd, hSf = bottom.gpu_data, top.gpu_data, self.blobScale.gpu_data, self.blobScale.gpu_diff
        n = bottom.count()
        cuda.copy(n, hB, hT)
        cuda.channel_max(nOuter * nInner, nOuter, nCh, nInner, hT, hSd)
        cuda.channel_sub(n, nOuter, nCh, nInner, hSd, hT)
        cuda.exp(n, hT, hT)
        cuda.channel_sum(nOuter * nInner, nOuter, nCh, nInner, hT, hSf)
        if self.algorithm == "LOG":
            cuda.log(nOuter * nInner, hSf, hSf)
            cuda.add(nOuter * nInner, hSd, hSf, hSd)
            cuda.copy(n, hB, hT)
            cuda.channel_sub(n, nOuter, nCh, nInner, hSd, hT)
        else:
            cuda.channel_div(n, nOuter, nCh, nInner, hSf, hT)

    def _backward_caffe(self, top, bottom):
        """SoftmaxLayer.cs:289-330 (the ACCURATE branch: inner1d(top_diff, top_data), subtract, multiply)."""
        cuda = self.cuda
        nOuter, nCh, nInner = self._dims
        n = top.count()
        if self.algorithm == "LOG":
            raise NotImplementedError("log-softmax gradient chain (channel_fillfrom over a reshaped scale blob)")
        cuda.copy(n, top.gpu_diff, bottom.gpu_diff)
        cuda.channel_dot(nOuter * nInner, nOuter, nCh, nInner, top.gpu_diff, top.gpu_data, self.blobScale.gpu_data)
        cuda.channel_sub(n, nOuter, nCh, nInner, self.blobScale.gpu_data, bottom.gpu_diff)
        cuda.mul(n, bottom.gpu_diff, top.gpu_data, bottom.gpu_diff)

    def Forward(self, bottom, top):
        if self.engine == "CAFFE":
            return self._forward_caffe(bottom, top)
        axis = self.axis % bottom.num_axes
        nN, nK, nH = bottom.count(0, axis), bottom.shape(axis), bottom.count(axis + 1)
        mode = SOFTMAX_MODE.INSTANCE if nH == 1 else SOFTMAX_MODE.CHANNEL
        top.ReshapeLike(bottom)
        self.cuda.SetTensorDesc(self.hBottomDesc, nN, nK, nH, 1, bottom.half)
        self.cuda.SetTensorDesc(self.hTopDesc, nN, nK, nH, 1, top.half)
        self.cuda.SoftmaxForward(self.hCudnn, SOFTMAX_ALGORITHM.ACCURATE, mode, 1.0, self.hBottomDesc, bottom.gpu_data, 0.0,
                                 self.hTopDesc, top.gpu_data)
        self._mode = mode

    def Backward(self, top, bottom):
        """SoftmaxLayer.cs:359-367: bottom.diff from top.data and top.diff (descriptors as set by Forward)."""
        if self.engine == "CAFFE":
            return self._backward_caffe(top, bottom)
        self.cuda.SoftmaxBackward(self.hCudnn, SOFTMAX_ALGORITHM.ACCURATE, self._mode, 1.0, self.hTopDesc, top.gpu_data, self.hTopDesc,
                                  top.gpu_diff, 0.0, self.hBottomDesc, bottom.gpu_diff)


class CausalSelfAttentionLayer:
    """MyCaffe.layers.gpt/layers.gpt/CausalSelfAttentionLayer.cs (setup :96-250, forward :526-628).

    ``enable_cuda_scaled_dot_product_attention`` selects the fused attention handle
    (ids 160-163); otherwise the explicit transpose / MatMul / scale / mask /
    softmax / MatMul chain runs, as in the reference.
    """

    def __init__(self, cuda, heads, embed, block_size, bias_term=True, enable_cuda_scaled_dot_product_attention=True,
                 enable_rotary_positional_embedding=False, rope_theta=10000.0, half=False, training=False,
                 fused_qkv_heads=False):
        self.training = training
        # three calls per forward instead of seventeen (ids with no counterpart in the reference): the fused QKV
        # projection writes q, k, v as (B,H,T,hs), rotated where the layer has a rotary embedding, the attention
        # handle writes its output head-merged and the output projection adds its bias in the GEMM's epilogue.
        # Inference, fused attention handle.
        self.fused_qkv_heads = fused_qkv_heads
        self.cuda, self.nHeads, self.nEmbed, self.nBlockSize = cuda, heads, embed, block_size
        self.nSize = embed // heads
        self.bias_term, self.half = bias_term, half
        self.enable_sdpa = enable_cuda_scaled_dot_product_attention
        self.enable_rope, self.rope_theta = enable_rotary_positional_embedding, rope_theta
        self.dfIgnoreVal = -1e29
        self.c_attn = InnerProductLayer(cuda, 3 * embed, bias_term, 2, half)
        self.c_proj = InnerProductLayer(cuda, embed, bias_term, 2, half, fused_bias=fused_qkv_heads)
        self.transpose = TransposeLayer(cuda, (0, 2, 1, 3))
        self.transposeQ = TransposeLayer(cuda, (0, 1, 3, 2))
        self.softmax = SoftmaxLayer(cuda, -1)
        names = "IpAttn Q K V Qt Kt Vt Kt1 AttA AttB Work Y".split()
        self.b = {n: Blob(cuda, half=half) for n in names}
        self.blobMask = Blob(cuda, (1, 1, block_size, block_size))
        mask = np.tril(np.ones((block_size, block_size), np.float32))  # fillMask :276-291
        self.blobMask.mutable_cpu_data = mask
        self.hCudnn = self.hAttn = self.hRope = 0
        self._set_for = None

    def Setup(self, bottom, w_attn, b_attn, w_proj, b_proj):
        self.c_attn.Setup(bottom, w_attn, b_attn)
        y = Blob(self.cuda, bottom.shape_, self.half)
        self.c_proj.Setup(y, w_proj, b_proj)
        y.Dispose()

    def _reshape(self, B, T):
        if self._set_for == (B, T):
            return
        if self.enable_sdpa:
            if not self.hCudnn:
                self.hCudnn = self.cuda.CreateCuDNN()
                self.hAttn = self.cuda.CreateAttn()
            self.cuda.SetAttn(self.hCudnn, self.hAttn, 0, self.training, B, self.nBlockSize, self.nHeads, self.nSize, 0.0)
        if self.enable_rope:
            if self.hRope:
                self.cuda.FreeRope(self.hRope)
            self.hRope = self.cuda.CreateRope(0, 0, B * T * self.nEmbed, B, T, self.nHeads, self.nSize, self.rope_theta)
        if T != self.nBlockSize and not self.enable_sdpa:
            m = Blob(self.cuda, (1, 1, T, T))
            m.mutable_cpu_data = np.tril(np.ones((T, T), np.float32))
            self.blobMaskT = m
        self._set_for = (B, T)

    def Forward(self, blobX, top):
        B, T, C = blobX.shape_[:3]
        if T > self.nBlockSize:
            raise ValueError("sequence longer than block_size")
        self._reshape(B, T)
        b, cuda, H, hs = self.b, self.cuda, self.nHeads, self.nSize
        if self.fused_qkv_heads:
            if not self.enable_sdpa or self.training:
                raise ValueError("fused_qkv_heads needs the fused attention handle, inference mode")
            for name in ("Qt", "Kt", "Vt"):
                b[name].Reshape(B, H, T, hs)
            ip = self.c_attn
            cuda.QkvProjHeads(B, T, H, hs, blobX.gpu_data, ip.blobs[0].gpu_data, ip.blobs[1].gpu_data if ip.bias_term else 0,
                              b["Qt"].gpu_data, b["Kt"].gpu_data, b["Vt"].gpu_data, self.hRope)
            mask = self.blobMask
            if T != self.nBlockSize:
                if getattr(self, "_sdpa_mask_T", None) != T:
                    self.blobMaskSdpa = Blob(cuda, (1, 1, T, T))
                    self.blobMaskSdpa.mutable_cpu_data = np.tril(np.ones((T, T), np.float32))
                    self._sdpa_mask_T = T
                mask = self.blobMaskSdpa
            b["Y"].Reshape(B, T, C)
            cuda.AttnScaledDotProductForward(self.hCudnn, self.hAttn, T, b["Qt"].gpu_data, b["Kt"].gpu_data, b["Vt"].gpu_data,
                                             mask.gpu_data, b["Y"].gpu_data, False, T, True)
            self.c_proj.Forward(b["Y"], top)
            return
        # q, k, v = self.c_attn(x).split(self.n_embd, dim=2)
        self.c_attn.Forward(blobX, b["IpAttn"])
        for name in "QKV":
            b[name].Reshape(B, T, H, hs)
        nCount = b["Q"].count()
        ip = b["IpAttn"]
        cuda.channel_copy(nCount, ip.num, ip.channels, 3, self.nEmbed, 0, ip.gpu_data, b["Q"].gpu_data, DIR.FWD)
        cuda.channel_copy(nCount, ip.num, ip.channels, 3, self.nEmbed, 1, ip.gpu_data, b["K"].gpu_data, DIR.FWD)
        cuda.channel_copy(nCount, ip.num, ip.channels, 3, self.nEmbed, 2, ip.gpu_data, b["V"].gpu_data, DIR.FWD)
        if self.hRope:
            cuda.RopeForward(self.hRope, b["Q"].count(), b["Q"].gpu_data, b["Q"].gpu_data)
            cuda.RopeForward(self.hRope, b["K"].count(), b["K"].gpu_data, b["K"].gpu_data)
        # (B, T, nh, hs) -> (B, nh, T, hs)
        self.transpose.Forward(b["Q"], b["Qt"])
        self.transpose.Forward(b["K"], b["Kt"])
        self.transpose.Forward(b["V"], b["Vt"])
        if self.enable_sdpa:
            b["Work"].ReshapeLike(b["Vt"])
            mask = self.blobMask
            if T != self.nBlockSize:
                # the handle reads a (1,1,T,T) mask for the block size it is run with
                if getattr(self, "_sdpa_mask_T", None) != T:
                    self.blobMaskSdpa = Blob(cuda, (1, 1, T, T))
                    self.blobMaskSdpa.mutable_cpu_data = np.tril(np.ones((T, T), np.float32))
                    self._sdpa_mask_T = T
                mask = self.blobMaskSdpa
            cuda.AttnScaledDotProductForward(self.hCudnn, self.hAttn, T, b["Qt"].gpu_data, b["Kt"].gpu_data, b["Vt"].gpu_data,
                                             mask.gpu_data, b["Work"].gpu_data, False)
        else:
            self.transposeQ.Forward(b["Kt"], b["Kt1"])
            dfScale = 1.0 / math.sqrt(hs)
            b["AttA"].MatMul(b["Qt"], b["Kt1"], bReshape=True)
            b["AttA"].scale_data(dfScale)
            mask = self.blobMask if T == self.nBlockSize else self.blobMaskT
            cuda.mask(b["AttA"].count(), mask.count(), 0.0, self.dfIgnoreVal, b["AttA"].gpu_data, mask.gpu_data, b["AttA"].gpu_data)
            self.softmax.Forward(b["AttA"], b["AttB"])
            b["Work"].MatMul(b["AttB"], b["Vt"], bReshape=True)
        # y.transpose(1, 2).contiguous().view(B, T, C)
        self.transpose.Forward(b["Work"], b["Y"])
        self._y_shape = list(b["Y"].shape_)
        b["Y"].Reshape(B, T, C)
        self.c_proj.Forward(b["Y"], top)

    def Backward(self, top, blobX):
        """CausalSelfAttentionLayer.cs:641-747: top.gpu_diff -> blobX.gpu_diff, parameter gradients accumulate in the
        InnerProduct weight diffs.  Fused handle: its backward call gets mask handle 0, as there.  Explicit chain: the
        two MatMulGrad calls around the softmax gradient (no dropout)."""
        b, cuda = self.b, self.cuda
        B, T, C = blobX.shape_[:3]
        self.c_proj.Backward(top, b["Y"])
        b["Y"].Reshape(*self._y_shape)
        self.transpose.Backward(b["Y"], b["Work"])
        b["Y"].CopyFrom(b["Work"], True, True)
        if self.enable_sdpa:
            cuda.AttnScaledDotProductBackward(self.hCudnn, self.hAttn, b["Qt"].gpu_data, b["Qt"].gpu_diff, b["Kt"].gpu_data,
                                              b["Kt"].gpu_diff, b["Vt"].gpu_data, b["Vt"].gpu_diff, 0, b["Y"].gpu_data, b["Y"].gpu_diff)
        else:
            # att' = y' @ v^T, vt' = att^T @ y'; softmax gradient; qt' = att' @ kt, kt1' = qt^T @ att' (scaled)
            b["Y"].MatMulGrad(b["AttB"], b["Vt"])
            self.softmax.Backward(b["AttB"], b["AttA"])
            b["AttA"].MatMulGrad(b["Qt"], b["Kt1"], 1.0 / math.sqrt(self.nSize))
            self.transposeQ.Backward(b["Kt1"], b["Kt"])
        self.transpose.Backward(b["Kt"], b["K"])
        self.transpose.Backward(b["Qt"], b["Q"])
        self.transpose.Backward(b["Vt"], b["V"])
        if self.hRope:
            cuda.RopeBackward(self.hRope, b["Q"].count(), b["Q"].gpu_data, b["Q"].gpu_diff, b["Q"].gpu_diff)
            cuda.RopeBackward(self.hRope, b["K"].count(), b["K"].gpu_data, b["K"].gpu_diff, b["K"].gpu_diff)
        nCount = b["Q"].count()
        ip = b["IpAttn"]
        cuda.channel_copy(nCount, ip.num, ip.channels, 3, self.nEmbed, 0, ip.gpu_diff, b["Q"].gpu_diff, DIR.BWD)
        cuda.channel_copy(nCount, ip.num, ip.channels, 3, self.nEmbed, 1, ip.gpu_diff, b["K"].gpu_diff, DIR.BWD)
        cuda.channel_copy(nCount, ip.num, ip.channels, 3, self.nEmbed, 2, ip.gpu_diff, b["V"].gpu_diff, DIR.BWD)
        b["Y"].Reshape(B, T, C)
        self.c_attn.Backward(ip, blobX)


class MultiheadAttentionLayer:
    """MyCaffe.layers.gpt/layers.gpt/MultiheadAttentionLayer.cs:643-811.  With ``enable_key_value_cache`` and the
    "position" layer option set, the explicit chain takes the reference's cached decode branch (:713-730, 759-777: one
    token per call, a loop over the cached positions); :meth:`CudaDnn.AttnDecodeForward` is the one-call replacement.

    ``Forward(q, k, v, mask)``: mask is ``None``, a (1,1,T,T) blob (causal), a
    (B,T_k) key-padding blob or a (B,T_q,T_k) blob; the last two take the
    mask_batch route, as in the reference (``fuse_batch_qk_mask`` sends the
    (B,T_q,T_k) mask to the fused handle instead, which the reference's handle
    cannot do).
    """

    def __init__(self, cuda, heads, embed, block_size, bias_term=True, enable_cuda_scaled_dot_product_attention=True,
                 enable_rotary_positional_embedding=False, rope_theta=10000.0, half=False, fuse_batch_qk_mask=False,
                 enable_key_value_cache=False):
        self.cuda, self.nHeads, self.nEmbed, self.nBlockSize = cuda, heads, embed, block_size
        self.fuse_batch_qk_mask = fuse_batch_qk_mask
        self.enable_kv_cache = enable_key_value_cache
        self.nSize = embed // heads
        self.half = half
        self.enable_sdpa = enable_cuda_scaled_dot_product_attention
        self.enable_rope, self.rope_theta = enable_rotary_positional_embedding, rope_theta
        self.c_attnQ = InnerProductLayer(cuda, embed, bias_term, 2, half)
        self.c_attnK = InnerProductLayer(cuda, embed, bias_term, 2, half)
        self.c_attnV = InnerProductLayer(cuda, embed, bias_term, 2, half)
        self.c_proj = InnerProductLayer(cuda, embed, bias_term, 2, half)
        self.transpose = TransposeLayer(cuda, (0, 2, 1, 3))
        self.transposeK = TransposeLayer(cuda, (0, 2, 1, 3))
        self.transposeQ = TransposeLayer(cuda, (0, 1, 3, 2))
        self.softmax = SoftmaxLayer(cuda, -1)
        self.b = {n: Blob(cuda, half=half) for n in "Q K V Qt Kt Vt Kt1 AttA AttB Work Y KeyCache ValCache Work2 Work3".split()}
        self.hCudnn = self.hAttn = self.hRope = 0
        self._set_for = None
        self.options = {}

    def SetLayerOption(self, name, value):
        self.options[name] = value

    def Setup(self, q, k, v, weights):
        """weights: dict with wq,bq,wk,bk,wv,bv,wo,bo ([out,in] matrices)."""
        self.c_attnQ.Setup(q, weights["wq"], weights.get("bq"))
        self.c_attnK.Setup(k, weights["wk"], weights.get("bk"))
        self.c_attnV.Setup(v, weights["wv"], weights.get("bv"))
        self.c_proj.Setup(q, weights["wo"], weights.get("bo"))

    def Forward(self, q, k, v, blobMask, top):
        cuda, H, hs, b = self.cuda, self.nHeads, self.nSize, self.b
        B, Tq, C = q.shape_[:3]
        Tk = k.shape_[1]
        nPos = int(self.options.get("position", -1))
        self.c_attnQ.Forward(q, b["Q"])
        self.c_attnK.Forward(k, b["K"])
        self.c_attnV.Forward(v, b["V"])
        b["Q"].Reshape(B, Tq, H, hs)
        b["K"].Reshape(B, Tk, H, hs)
        b["V"].Reshape(B, Tk, H, hs)
        if self.enable_rope:
            if not self.hRope:
                self.hRope = cuda.CreateRope(0, 0, B * self.nBlockSize * C, B, self.nBlockSize, H, hs, self.rope_theta)
            nFreqOffset = nPos * hs // 2 if nPos > 0 else -1
            cuda.RopeForward(self.hRope, b["Q"].count(), b["Q"].gpu_data, b["Q"].gpu_data, nFreqOffset)
            cuda.RopeForward(self.hRope, b["K"].count(), b["K"].gpu_data, b["K"].gpu_data, nFreqOffset)
        self.transpose.Forward(b["Q"], b["Qt"])
        self.transposeK.Forward(b["K"], b["Kt"])
        self.transposeK.Forward(b["V"], b["Vt"])
        is_qk_mask = (blobMask is not None and blobMask.num_axes == 4 and blobMask.num == 1 and blobMask.channels == 1
                      and blobMask.height == Tq and blobMask.width == Tk)
        full_mask = blobMask is not None and not is_qk_mask and blobMask.count() == B * Tq * Tk and Tq > 1
        if self.enable_sdpa and (not full_mask or self.fuse_batch_qk_mask):
            if self._set_for != B:
                if not self.hCudnn:
                    self.hCudnn = cuda.CreateCuDNN()
                    self.hAttn = cuda.CreateAttn()
                cuda.SetAttn(self.hCudnn, self.hAttn, 0, False, B, self.nBlockSize, H, hs, 0.0)
                self._set_for = B
            b["Work"].ReshapeLike(b["Qt"])
            cuda.AttnScaledDotProductForward(self.hCudnn, self.hAttn, Tq, b["Qt"].gpu_data, b["Kt"].gpu_data, b["Vt"].gpu_data,
                                             blobMask.gpu_data if blobMask is not None else 0, b["Work"].gpu_data,
                                             2 if full_mask else (not is_qk_mask), Tk if Tk != Tq else None)
        else:
            # the fused handle only understands (1,1,T,T) or (B,T) masks (attn.cu:544-556); a
            # (B,T_q,T_k) mask goes through the explicit chain (MultiheadAttentionLayer.cs:733-742)
            self.transposeQ.Forward(b["Kt"], b["Kt1"])
            dfScale = 1.0 / math.sqrt(hs)
            cached = nPos >= 0 and self.enable_kv_cache
            if cached:
                # one token: append its key / value to the caches (sized for the block size at the first call, as the
                # layer's reshape does), then one MatMul per cached position (:713-730)
                for name in ("KeyCache", "ValCache"):
                    if b[name]._capacity == 0:
                        b[name].Reshape(B, H, self.nBlockSize, hs)
                b["KeyCache"].Reshape(nPos + 1, H, hs, 1)
                b["ValCache"].Reshape(nPos + 1, H, 1, hs)
                nK, nV = b["Kt1"].count(), b["Vt"].count()
                cuda.copy(nK, b["Kt1"].gpu_data, b["KeyCache"].gpu_data, 0, nPos * nK)
                cuda.copy(nV, b["Vt"].gpu_data, b["ValCache"].gpu_data, 0, nPos * nV)
                b["AttA"].Reshape(1, H, 1, nPos + 1)
                for i in range(nPos + 1):
                    cuda.copy(nK, b["KeyCache"].gpu_data, b["Kt1"].gpu_data, i * nK, 0)
                    b["Work2"].MatMul(b["Qt"], b["Kt1"], True)
                    b["Work2"].scale_data(dfScale)
                    cuda.channel_copy(b["Work2"].count(), 1, H, nPos + 1, 1, i, b["AttA"].gpu_data, b["Work2"].gpu_data, DIR.BWD)
            else:
                b["AttA"].MatMul(b["Qt"], b["Kt1"], bReshape=True)
                b["AttA"].scale_data(dfScale)
                if blobMask is not None:
                    if is_qk_mask:
                        cuda.mask(b["AttA"].count(), blobMask.count(), 0.0, -1e29, b["AttA"].gpu_data, blobMask.gpu_data, b["AttA"].gpu_data)
                    else:
                        cuda.mask_batch(b["AttA"].count(), b["AttA"].num, blobMask.count(), 0.0, -1e29, b["AttA"].gpu_data,
                                        blobMask.gpu_data, b["AttA"].gpu_data)
            self.softmax.Forward(b["AttA"], b["AttB"])
            if cached:
                # y = sum over the cached positions of weight_i * v_i, one MatMul and one add per position (:759-777)
                b["Work"].Reshape(1, H, 1, hs)
                b["Work3"].Reshape(1, H, 1, 1)
                b["Work2"].Reshape(1, H, 1, hs)
                nV = b["Vt"].count()
                for i in range(nPos + 1):
                    cuda.copy(nV, b["ValCache"].gpu_data, b["Vt"].gpu_data, i * nV, 0)
                    cuda.channel_copy(b["Work3"].count(), 1, H, nPos + 1, 1, i, b["AttB"].gpu_data, b["Work3"].gpu_data, DIR.FWD)
                    b["Work2"].MatMul(b["Work3"], b["Vt"], True)
                    if i == 0:
                        cuda.copy(b["Work"].count(), b["Work2"].gpu_data, b["Work"].gpu_data)
                    else:
                        cuda.add(b["Work"].count(), b["Work2"].gpu_data, b["Work"].gpu_data, b["Work"].gpu_data)
            else:
                b["Work"].MatMul(b["AttB"], b["Vt"], bReshape=True)
        self.transpose.Forward(b["Work"], b["Y"])
        b["Y"].Reshape(B, Tq, C)
        self.c_proj.Forward(b["Y"], top)


class LayerNormLayer:
    """MyCaffe.layers.gpt/layers.gpt/LayerNormLayer.cs.  ``enable_cuda_impl`` runs the LayerNorm handle (ids 970-976;
    reshape :153-166, forward :211-212, backward :285-286); otherwise the explicit chain of :223-264 runs (channel_mean,
    channel_fillfrom, sub, powx, channel_mean, add_scalar, sqrt, channel_fillfrom, div)."""

    def __init__(self, cuda, epsilon=1e-10, enable_cuda_impl=True):
        self.cuda, self.epsilon, self.enable_cuda_impl = cuda, epsilon, enable_cuda_impl
        self.hLayerNorm = 0
        self._shape = None
        self.b = {n: Blob(cuda) for n in "Mu Xmu XmuSq Var Stdev StdevFull Work".split()}

    def _reshape(self, bottom):
        nAxis = len(bottom.shape_) - 1
        self.nCount = bottom.count()
        self.nOuterNum, self.nChannels, self.nInnerNum = bottom.shape_[0], bottom.count(1, nAxis), bottom.count(nAxis)
        if self._shape == bottom.shape_:
            return
        if self.enable_cuda_impl:
            if self.hLayerNorm:
                self.cuda.FreeLayerNorm(self.hLayerNorm)
            self.hLayerNorm = self.cuda.CreateLayerNorm(0, self.nCount, self.nOuterNum, self.nChannels, self.nInnerNum, self.epsilon)
        else:
            for n in ("Xmu", "XmuSq", "StdevFull"):
                self.b[n].ReshapeLike(bottom)
            for n in ("Mu", "Var", "Stdev"):
                self.b[n].Reshape(self.nOuterNum, self.nChannels, 1, 1)
        self._shape = list(bottom.shape_)

    def Forward(self, bottom, top):
        self._reshape(bottom)
        top.ReshapeLike(bottom)
        cuda, b = self.cuda, self.b
        if self.enable_cuda_impl:
            cuda.LayerNormForward(self.hLayerNorm, bottom.gpu_data, top.gpu_data)
            return
        n, o, c, i = self.nCount, self.nOuterNum, self.nChannels, self.nInnerNum
        cuda.channel_mean(n, o, c, i, bottom.gpu_data, b["Mu"].gpu_data)
        cuda.channel_fillfrom(n, o, c, i, b["Mu"].gpu_data, b["Xmu"].gpu_data, DIR.FWD)
        cuda.sub(n, bottom.gpu_data, b["Xmu"].gpu_data, b["Xmu"].gpu_data)
        cuda.powx(n, b["Xmu"].gpu_data, 2.0, b["XmuSq"].gpu_data)
        cuda.channel_mean(n, o, c, i, b["XmuSq"].gpu_data, b["Var"].gpu_data)
        cuda.add_scalar(o * c, self.epsilon, b["Var"].gpu_data)
        cuda.sqrt(o * c, b["Var"].gpu_data, b["Stdev"].gpu_data)
        cuda.channel_fillfrom(n, o, c, i, b["Stdev"].gpu_data, b["StdevFull"].gpu_data, DIR.FWD)
        cuda.div(n, b["Xmu"].gpu_data, b["StdevFull"].gpu_data, top.gpu_data)

    def Backward(self, top, bottom):
        if self.enable_cuda_impl:
            self.cuda.LayerNormBackward(self.hLayerNorm, top.gpu_data, top.gpu_diff, bottom.gpu_diff)
            return
        # LayerNormLayer.cs:292-320, the layer's own chain: dx = (dy - (y * mean(y * dy) + mean(dy))) / (std + eps)
        cuda, b = self.cuda, self.b
        n, o, c, i = self.nCount, self.nOuterNum, self.nChannels, self.nInnerNum
        b["Work"].ReshapeLike(top)
        cuda.mul(n, top.gpu_data, top.gpu_diff, b["Work"].gpu_data)
        cuda.channel_mean(n, o, c, i, b["Work"].gpu_data, b["Var"].gpu_diff)
        cuda.channel_mean(n, o, c, i, top.gpu_diff, b["Stdev"].gpu_diff)
        cuda.channel_fillfrom(n, o, c, i, b["Var"].gpu_diff, b["StdevFull"].gpu_diff, DIR.FWD)
        cuda.mul(n, top.gpu_data, b["StdevFull"].gpu_diff, b["Work"].gpu_data)
        cuda.channel_fillfrom(n, o, c, i, b["Stdev"].gpu_diff, b["StdevFull"].gpu_diff, DIR.FWD)
        cuda.add(n, b["Work"].gpu_data, b["StdevFull"].gpu_diff, b["Work"].gpu_data)
        cuda.sub(n, top.gpu_diff, b["Work"].gpu_data, b["Work"].gpu_data)
        cuda.add_scalar(b["StdevFull"].count(), self.epsilon, b["StdevFull"].gpu_data)
        cuda.div(n, b["Work"].gpu_data, b["StdevFull"].gpu_data, bottom.gpu_diff)


class RMSNormLayer:
    """MyCaffe.layers.gpt/layers.gpt/RMSNormLayer.cs:96-180, the layer's own chain: powx(2), channel_mean, sqrt(+eps),
    invert, channel_duplicate, mul, and with weights channel_copyall + mul.  ``fused`` replaces the chain by the
    single call RMSNORM_FWD (id 2002), which has no counterpart in the reference."""

    def __init__(self, cuda, epsilon=1e-5, enable_weights=True, fused=False):
        self.cuda, self.epsilon, self.enable_weights, self.fused = cuda, epsilon, enable_weights, fused
        self.blobs = []
        self.b = {n: Blob(cuda) for n in "Rms Rms1 Out Rms1Full".split()}

    def Setup(self, bottom, weight=None):
        nAxis = len(bottom.shape_) - 1
        if self.enable_weights:
            w = Blob(self.cuda, (bottom.count(nAxis),))
            w.mutable_cpu_data = np.ones(bottom.count(nAxis), np.float32) if weight is None else weight
            self.blobs = [w]

    def Forward(self, bottom, top):
        cuda, b = self.cuda, self.b
        nAxis = len(bottom.shape_) - 1
        n, inner = bottom.count(), bottom.count(nAxis)
        channels, outer = bottom.shape_[nAxis - 1], bottom.count(0, nAxis - 1)
        top.ReshapeLike(bottom)
        if self.fused:
            cuda.RmsNormForward(outer * channels, inner, bottom.gpu_data, self.blobs[0].gpu_data if self.enable_weights else 0,
                                top.gpu_data, self.epsilon)
            return
        b["Rms"].Reshape(outer, channels, 1, 1)
        b["Rms1"].Reshape(outer, channels, 1, 1)
        b["Out"].ReshapeLike(bottom)
        b["Rms1Full"].ReshapeLike(bottom)
        cuda.powx(n, bottom.gpu_data, 2.0, top.gpu_data)
        cuda.channel_mean(n, outer, channels, inner, top.gpu_data, b["Rms"].gpu_data)
        cuda.sqrt(b["Rms"].count(), b["Rms"].gpu_data, b["Rms"].gpu_data, self.epsilon)
        cuda.invert(b["Rms1"].count(), b["Rms"].gpu_data, b["Rms1"].gpu_data)
        cuda.channel_duplicate(n, outer * channels, 1, inner, b["Rms1"].gpu_data, b["Rms1Full"].gpu_data)
        cuda.mul(n, bottom.gpu_data, b["Rms1Full"].gpu_data, b["Out"].gpu_data)
        if self.enable_weights:
            cuda.channel_copyall(n, outer * channels, 1, inner, self.blobs[0].gpu_data, b["Out"].gpu_diff)
            cuda.mul(n, b["Out"].gpu_diff, b["Out"].gpu_data, top.gpu_data)
        else:
            top.CopyFrom(b["Out"])
        self._dims = (n, outer, channels, inner)

    def Backward(self, top, bottom, freeze_learning=False):
        """RMSNormLayer.cs:189-232, the layer's own chain (after a Forward through the chain): top.diff -> bottom.diff and,
        with weights, the weight gradient through channel_sum (which, as there, keeps the sums of the first batch
        entry: the call passes outer = batch and a gradient blob of `inner` values)."""
        if self.fused:
            raise NotImplementedError("the fused forward call keeps none of the chain's intermediates")
        cuda, b = self.cuda, self.b
        n, outer, channels, inner = self._dims
        if self.enable_weights:
            if not freeze_learning:
                cuda.mul(n, top.gpu_diff, b["Out"].gpu_data, b["Out"].gpu_data)
                cuda.channel_sum(n, outer, channels, inner, b["Out"].gpu_data, self.blobs[0].gpu_diff)
            cuda.mul(n, top.gpu_diff, b["Out"].gpu_diff, b["Out"].gpu_diff)
        # (without weights the reference reads Out's gradient here although nothing has written it; same here)
        # x6 = x * x5 -> dx and dx5
        cuda.mul(n, b["Out"].gpu_diff, b["Rms1Full"].gpu_data, bottom.gpu_diff)
        cuda.mul(n, b["Out"].gpu_diff, bottom.gpu_data, b["Rms1Full"].gpu_diff)
        cuda.channel_sumEx(n, outer, channels, inner, b["Rms1Full"].gpu_diff, b["Rms1"].gpu_diff, False, DIR.FWD)
        # x5 = 1 / x4 -> dx4
        cuda.powx(b["Rms"].count(), b["Rms"].gpu_data, 2.0, b["Rms"].gpu_diff)
        cuda.invert(b["Rms"].count(), b["Rms"].gpu_diff, b["Rms"].gpu_diff, 0, 0, -1)
        cuda.mul(b["Rms1"].count(), b["Rms1"].gpu_diff, b["Rms"].gpu_diff, b["Rms"].gpu_diff)
        # x4 = sqrt(x2 + eps) -> dx2
        cuda.invert(b["Rms1"].count(), b["Rms"].gpu_data, b["Rms1"].gpu_diff, 0, 0, 1, 2)
        cuda.mul(b["Rms"].count(), b["Rms1"].gpu_diff, b["Rms"].gpu_diff, b["Rms"].gpu_diff)
        # x2 = mean(x1) -> dx1
        cuda.channel_duplicate(n, outer * channels, 1, inner, b["Rms"].gpu_diff, b["Rms1Full"].gpu_diff)
        cuda.scal(b["Rms1Full"].count(), 1.0 / inner, b["Rms1Full"].gpu_diff)
        # x1 = x^2 -> dx, and the sum of both paths
        cuda.scale(n, 2.0, bottom.gpu_data, b["Out"].gpu_diff)
        cuda.mul(n, b["Out"].gpu_diff, b["Rms1Full"].gpu_diff, b["Out"].gpu_diff)
        cuda.add(n, b["Out"].gpu_diff, bottom.gpu_diff, bottom.gpu_diff)


class ActivationLayer:
    """ReLU (MyCaffe/layers/ReLULayer.cs), GELU (MyCaffe.layers.gpt/layers.gpt/GeluLayer.cs, ``enable_bert_version``) or
    SiLU (MyCaffe/layers/SiLULayer.cs) as TransformerBlockLayer selects them (TransformerBlockLayer.cs:316-337)."""

    def __init__(self, cuda, kind="relu"):
        if kind not in ("relu", "gelu", "gelu_bert", "silu"):
            raise ValueError(kind)
        self.cuda, self.kind = cuda, kind
        self.blobX = Blob(cuda)     # GeluLayer.cs:84-87: the input is kept when the layer runs in place

    def Forward(self, bottom, top):
        top.ReshapeLike(bottom)
        n = bottom.count()
        hBottom = bottom.gpu_data
        if self.kind != "relu" and bottom.gpu_data == top.gpu_data:
            self.blobX.CopyFrom(bottom)
            hBottom = self.blobX.gpu_data
        if self.kind == "relu":
            self.cuda.relu_fwd(n, hBottom, top.gpu_data, 0.0)
        elif self.kind == "silu":
            self.cuda.silu_fwd(n, hBottom, top.gpu_data)
        else:
            self.cuda.gelu_fwd(n, hBottom, top.gpu_data, self.kind == "gelu_bert")

    def Backward(self, top, bottom):
        """ReLULayer.cs:203, GeluLayer.cs:110-121, SiLULayer.cs backward."""
        n = bottom.count()
        hBottomData = bottom.gpu_data
        if top.gpu_data == bottom.gpu_data:
            hBottomData = self.blobX.gpu_data
        if self.kind == "relu":
            self.cuda.relu_bwd(n, top.gpu_diff, top.gpu_data, bottom.gpu_diff, 0.0)
        elif self.kind == "silu":
            self.cuda.silu_bwd(n, top.gpu_diff, top.gpu_data, bottom.gpu_diff, hBottomData)
        else:
            self.cuda.gelu_bwd(n, top.gpu_diff, top.gpu_data, bottom.gpu_diff, hBottomData, self.kind == "gelu_bert")


class TransformerBlockLayer:
    """MyCaffe.layers.gpt/layers.gpt/TransformerBlockLayer.cs, block types CAUSAL_SELF_ATTENTION and ENCODER (setup
    :99-170, 252-340, forward :800-902): x + attn(ln1(x)), then + proj(act(fc(ln2(.)))).  The ENCODER type attends
    through MultiheadAttentionLayer(x_1, x_1, x_1, mask), the form the Llama models built by LlamaModelBuilder use
    (rotary embedding, key / value cache, "position" layer option).  Dropout is the identity at inference."""

    def __init__(self, cuda, heads, embed, block_size, activation="relu", bias_term=True, epsilon=1e-10,
                 enable_cuda_scaled_dot_product_attention=True, training=False, enable_llama_style_head=False, hidden_dim=0,
                 multiple_of=64, enable_layernorm_cuda_impl=True, fused_rmsnorm=False, block_type="causal_self_attention",
                 enable_key_value_cache=False):
        if block_type not in ("causal_self_attention", "encoder"):
            raise ValueError(block_type)
        self.cuda = cuda
        self.block_type = block_type
        self.llama = enable_llama_style_head
        if self.llama:
            # RMSNorm, rotary attention without bias, SiLU-gated MLP (TransformerBlockLayer.cs:86-98, 239-247, 860-875)
            self.norm1 = RMSNormLayer(cuda, epsilon, True, fused_rmsnorm)
            self.norm2 = RMSNormLayer(cuda, epsilon, True, fused_rmsnorm)
            if hidden_dim == 0:
                hidden_dim = 2 * (4 * embed) // 3
                hidden_dim = multiple_of * ((hidden_dim + multiple_of - 1) // multiple_of)
        else:
            self.norm1 = LayerNormLayer(cuda, epsilon, enable_layernorm_cuda_impl)
            self.norm2 = LayerNormLayer(cuda, epsilon, enable_layernorm_cuda_impl)
            hidden_dim = hidden_dim or 4 * embed
        if block_type == "encoder":
            self.attn1 = MultiheadAttentionLayer(cuda, heads, embed, block_size, bias_term, enable_cuda_scaled_dot_product_attention,
                                                 enable_rotary_positional_embedding=self.llama,
                                                 enable_key_value_cache=enable_key_value_cache)
        else:
            self.attn1 = CausalSelfAttentionLayer(cuda, heads, embed, block_size, bias_term, enable_cuda_scaled_dot_product_attention,
                                                  enable_rotary_positional_embedding=self.llama, training=training)
        self.fc1 = InnerProductLayer(cuda, hidden_dim, bias_term, 2)
        self.fc2 = InnerProductLayer(cuda, hidden_dim, bias_term, 2) if self.llama else None
        self.proj = InnerProductLayer(cuda, embed, bias_term, 2)
        self.act = ActivationLayer(cuda, activation)
        self.b = {n: Blob(cuda) for n in "Norm1 Attn1 X Norm2 NormA Mlp1 Mlp2 Mlp3 MlpOut".split()}

    def Setup(self, bottom, p):
        """``p``: attn_weight, attn_bias, attn_proj_weight, attn_proj_bias (ENCODER type: wq, bq, wk, bk, wv, bv, wo, bo),
        fc_weight, fc_bias, proj_weight, proj_bias; Llama style also fc2_weight, rms1_weight, rms2_weight."""
        if self.block_type == "encoder":
            self.attn1.Setup(bottom, bottom, bottom, p)
        else:
            self.attn1.Setup(bottom, p["attn_weight"], p.get("attn_bias"), p["attn_proj_weight"], p.get("attn_proj_bias"))
        self.fc1.Setup(bottom, p["fc_weight"], p.get("fc_bias"))
        if self.llama:
            self.fc2.Setup(bottom, p["fc2_weight"], p.get("fc2_bias"))
            self.norm1.Setup(bottom, p.get("rms1_weight"))
            self.norm2.Setup(bottom, p.get("rms2_weight"))
        hidden = Blob(self.cuda, bottom.shape_[:2] + [self.fc1.N])
        self.proj.Setup(hidden, p["proj_weight"], p.get("proj_bias"))
        hidden.Dispose()

    def SetLayerOption(self, name, value):
        """Layer options reach the attention layer (TransformerBlockLayer.cs SetLayerOption override)."""
        if self.block_type == "encoder":
            self.attn1.SetLayerOption(name, value)

    def Forward(self, blobX, top, blobXMask=None):
        b, cuda = self.b, self.cuda
        nCount = blobX.count()
        self.norm1.Forward(blobX, b["Norm1"])
        if self.block_type == "encoder":
            self.attn1.Forward(b["Norm1"], b["Norm1"], b["Norm1"], blobXMask, b["Attn1"])
        else:
            self.attn1.Forward(b["Norm1"], b["Attn1"])
        b["X"].ReshapeLike(blobX)
        cuda.add(nCount, blobX.gpu_data, b["Attn1"].gpu_data, b["X"].gpu_data)
        self.norm2.Forward(b["X"], b["Norm2"])
        self.fc1.Forward(b["Norm2"], b["Mlp1"])
        self.act.Forward(b["Mlp1"], b["Mlp1"])
        blobMlp = b["Mlp1"]
        if self.llama:
            self.fc2.Forward(b["Norm2"], b["Mlp2"])
            b["Mlp3"].ReshapeLike(b["Mlp1"])
            cuda.mul(b["Mlp1"].count(), b["Mlp1"].gpu_data, b["Mlp2"].gpu_data, b["Mlp3"].gpu_data)
            blobMlp = b["Mlp3"]
        self.proj.Forward(blobMlp, b["MlpOut"])
        top.ReshapeLike(blobX)
        cuda.add(nCount, b["X"].gpu_data, b["MlpOut"].gpu_data, top.gpu_data)

    def Backward(self, top, blobX):
        """TransformerBlockLayer.cs:924-1040, CAUSAL_SELF_ATTENTION block: top.gpu_diff -> blobX.gpu_diff."""
        if self.block_type != "causal_self_attention":
            raise NotImplementedError("backward is mirrored for the CAUSAL_SELF_ATTENTION block type")
        b, cuda = self.b, self.cuda
        nCount = blobX.count()
        cuda.copy(nCount, top.gpu_diff, b["MlpOut"].gpu_diff)
        cuda.copy(nCount, top.gpu_diff, b["X"].gpu_diff)
        self.proj.Backward(b["MlpOut"], b["Mlp3"] if self.llama else b["Mlp1"])
        if self.llama:
            # gate: Mlp3 = silu(fc1) * fc2; the gradient through fc2 waits in NormA's data until fc1's has arrived
            n1 = b["Mlp1"].count()
            cuda.mul(n1, b["Mlp3"].gpu_diff, b["Mlp2"].gpu_data, b["Mlp1"].gpu_diff)
            cuda.mul(n1, b["Mlp3"].gpu_diff, b["Mlp1"].gpu_data, b["Mlp2"].gpu_diff)
            self.fc2.Backward(b["Mlp2"], b["Norm2"])
            b["NormA"].ReshapeLike(b["Norm2"])
            cuda.copy(b["Norm2"].count(), b["Norm2"].gpu_diff, b["NormA"].gpu_data)
        self.act.Backward(b["Mlp1"], b["Mlp1"])
        self.fc1.Backward(b["Mlp1"], b["Norm2"])
        if self.llama:
            cuda.add(b["Norm2"].count(), b["NormA"].gpu_data, b["Norm2"].gpu_diff, b["Norm2"].gpu_diff)
        # x_2 = ln_2(xB): keep xB's own gradient aside, add the one that comes through the norm
        b["Attn1"].CopyFrom(b["X"], True)
        self.norm2.Backward(b["Norm2"], b["X"])
        cuda.add(nCount, b["Attn1"].gpu_diff, b["X"].gpu_diff, b["X"].gpu_diff)
        b["Attn1"].CopyFrom(b["X"], True)
        self.attn1.Backward(b["Attn1"], b["Norm1"])
        self.norm1.Backward(b["Norm1"], blobX)
        cuda.add(nCount, b["X"].gpu_diff, blobX.gpu_diff, blobX.gpu_diff)
