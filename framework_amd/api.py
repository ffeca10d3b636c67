"""Host-side mirror of the reference's TypeScript API for the matmul path.

`bind(native)` returns a namespace with Tensor, Linear, ReLU, Adam, mseLoss,
crossEntropyLoss ... whose methods forward tensor ids to `native`, an object
with the reference's N-API export names (src/tensor.ts, src/nn.ts,
src/optimizer.ts, src/module.ts).  The default namespace of the package is
bound to the HIP backend; tests bind a second one to the CPU oracle and run
the same script against both.
"""
import math
from types import SimpleNamespace

import numpy as np


def bind(native):
    class Tensor:  # src/tensor.ts:9-252
        def __init__(self, id, shape=None):
            self._id = id
            # the reference asks native.tensorShape(id) here when no shape is given; this mirror asks on first use
            # (most results of a training step are passed on by id and never asked for their shape)
            self._known_shape = list(shape) if shape is not None else None

        @property
        def _shape(self):
            if self._known_shape is None:
                self._known_shape = [int(s) for s in native.tensorShape(self._id)]
            return self._known_shape

        @property
        def shape(self):
            return self._shape

        @property
        def size(self):
            n = 1
            for s in self._shape:
                n *= s
            return n

        @property
        def dims(self):
            return len(self._shape)

        # gradient
        @property
        def grad(self):
            gid = native.getGrad(self._id)
            return None if gid is None else Tensor(gid)

        def backward(self):
            native.backward(self._id)

        def requiresGrad(self):
            return native.getGrad(self._id) is not None

        # data transfer
        def toFloat32(self):
            return native.toFloat32(self._id)

        def item(self):
            return native.getScalar(self._id)

        def numpy(self):
            return np.asarray(self.toFloat32(), dtype=np.float32).reshape(self._shape)

        def free(self):
            native.freeTensor(self._id)

        # creation
        @staticmethod
        def fromFloat32(data, shape):
            return Tensor(native.fromFloat32(np.asarray(data, dtype=np.float32), list(shape)), shape)

        @staticmethod
        def zeros(shape):
            return Tensor(native.zeros(list(shape)), shape)

        @staticmethod
        def ones(shape):
            return Tensor(native.ones(list(shape)), shape)

        @staticmethod
        def rand(shape):  # src/tensor.ts rand -> native.randTensor, uniform [0, 1)
            return Tensor(native.randTensor(list(shape)), shape)

        @staticmethod
        def randn(shape):
            return Tensor(native.randnTensor(list(shape)), shape)

        # elementwise (src/tensor.ts:101-133): a number becomes a [1] tensor for
        # add/sub and a scalar multiply for mul
        def add(self, other):
            if isinstance(other, (int, float)):
                other = Tensor.fromFloat32([other], [1])
            return Tensor(native.add(self._id, other._id))

        def sub(self, other):
            if isinstance(other, (int, float)):
                other = Tensor.fromFloat32([other], [1])
            return Tensor(native.sub(self._id, other._id))

        def mul(self, other):
            if isinstance(other, (int, float)):
                return Tensor(native.mulScalar(self._id, other))
            return Tensor(native.mul(self._id, other._id))

        def neg(self):
            return Tensor(native.neg(self._id))

        def relu(self):
            return Tensor(native.relu(self._id))

        def gelu(self):  # src/nn.ts gelu() -> native.gelu
            return Tensor(native.gelu(self._id))

        def sum(self, dim=None):
            return Tensor(native.sumAll(self._id) if dim is None else native.sumOp(self._id, dim))

        def mean(self, dim=None):
            return Tensor(native.meanAll(self._id) if dim is None else native.meanOp(self._id, dim))

        def view(self, *shape):
            return Tensor(native.view(self._id, list(shape)))

        def permute(self, *dims):
            return Tensor(native.permute(self._id, list(dims)))

        def contiguous(self):
            return Tensor(native.contiguous(self._id))

        def exp(self):
            return Tensor(native.expOp(self._id))

        def log(self):
            return Tensor(native.logOp(self._id))

        def sigmoid(self):
            return Tensor(native.sigmoid(self._id))

        def pow(self, exponent):
            return Tensor(native.powOp(self._id, exponent))

        def div(self, other):
            return Tensor(native.div(self._id, other._id))

        def lt(self, other):
            return Tensor(native.lt(self._id, other._id))

        def eq(self, other):
            return Tensor(native.eqOp(self._id, other._id))

        def gt(self, other):
            return Tensor(native.gt(self._id, other._id))

        def isClose(self, other, tol=1e-5):
            return Tensor(native.isClose(self._id, other._id, tol))

        def max(self, dim):
            return Tensor(native.maxOp(self._id, dim))

        def matmul(self, other):  # src/tensor.ts:207-209
            return Tensor(native.matmul(self._id, other._id))

        def setRequiresGrad(self, requires):
            native.setRequiresGrad(self._id, requires)
            return self

    class Parameter:  # src/module.ts
        def __init__(self, value):
            self.value = value

    class Module:
        def parameters(self):
            out = []
            for v in self.__dict__.values():
                if isinstance(v, Parameter):
                    out.append(v)
                elif isinstance(v, Module):
                    out.extend(v.parameters())
                elif isinstance(v, (list, tuple)):
                    for m in v:
                        if isinstance(m, Module):
                            out.extend(m.parameters())
            return out

        def __call__(self, x):
            return self.forward(x)

    class Linear(Module):  # src/nn.ts:8-26: weight is [in, out], bound 1/sqrt(in) for both
        def __init__(self, inFeatures, outFeatures, weight=None, bias=None, fused=False, activation=None):
            self.inFeatures, self.outFeatures = inFeatures, outFeatures
            bound = 1.0 / math.sqrt(inFeatures)
            if weight is None:
                weight = np.random.uniform(-bound, bound, (inFeatures, outFeatures)).astype(np.float32)
            if bias is None:
                bias = np.random.uniform(-bound, bound, (outFeatures,)).astype(np.float32)
            self.weight = Parameter(Tensor.fromFloat32(weight, [inFeatures, outFeatures]).setRequiresGrad(True))
            self.bias = Parameter(Tensor.fromFloat32(bias, [outFeatures]).setRequiresGrad(True))
            # opt-in fused path, feature-detected like the reference's cuda-only ops
            self.fused = fused and hasattr(native, "linear")
            # None, "relu" or "gelu": applied by forward(); with the fused path it rides in native.linear
            self.activation = activation

        def forward(self, x):
            if self.fused:
                act = {None: 1, "relu": 2, "gelu": 3}[self.activation]  # MNI_EPI_BIAS / _RELU / _GELU
                return Tensor(native.linear(x._id, self.weight.value._id, self.bias.value._id, act))
            y = x.matmul(self.weight.value).add(self.bias.value)
            return y if self.activation is None else (y.relu() if self.activation == "relu" else y.gelu())

    class Embedding(Module):  # src/nn.ts:46-71: weight [vocab, dim], bound 1/sqrt(dim)
        def __init__(self, vocabSize, embedDim, weight=None):
            self.vocabSize, self.embedDim = vocabSize, embedDim
            bound = 1.0 / math.sqrt(embedDim)
            if weight is None:
                weight = np.random.uniform(-bound, bound, (vocabSize, embedDim)).astype(np.float32)
            self.weight = Parameter(Tensor.fromFloat32(weight, [vocabSize, embedDim]).setRequiresGrad(True))

        def forward(self, indices):
            batch, seqLen = len(indices), len(indices[0])
            flat = [int(i) for row in indices for i in row]
            return Tensor(native.embeddingForward(self.weight.value._id, flat, batch, seqLen))

        def forwardGpu(self, intBufId, batch, seqLen):
            return Tensor(native.embeddingForwardGpu(self.weight.value._id, intBufId, batch, seqLen))

    class ReLU(Module):
        def forward(self, x):
            return x.relu()

    class GELU(Module):
        def forward(self, x):
            return x.gelu()

    def mseLoss(pred, target, fused=False):  # src/nn.ts:161-165: mean(-1) twice
        if fused and hasattr(native, "mseLoss") and list(pred.shape) == list(target.shape):
            return Tensor(native.mseLoss(pred._id, target._id))  # opt-in: the same values from one pass
        diff = pred.sub(target)
        sq = diff.mul(diff)
        return Tensor(native.meanOp(Tensor(native.meanOp(sq._id, -1))._id, -1))

    def crossEntropyLoss(logits, targets):  # src/nn.ts:90-100
        V = logits.shape[-1]
        BT = logits.size // V
        flat = logits.view(BT, V)
        flat_targets = [int(t) for row in targets for t in (row if isinstance(row, (list, tuple, np.ndarray)) else [row])]
        return Tensor(native.crossEntropyLoss(flat._id, flat_targets))

    def crossEntropyLossGpu(logits, intBufId):  # src/nn.ts:102-105
        return Tensor(native.crossEntropyLossGpu(logits._id, intBufId))

    def dropout(x, rate=0.0, inference=False):  # src/nn.ts:85-88
        if inference or rate == 0:
            return x
        return Tensor(native.dropoutOp(x._id, rate, True))

    def residualLayerNorm(x, residual, gamma, beta, eps=1e-5):  # src/nn.ts:149-151
        return Tensor(native.residualLayernorm(x._id, residual._id, gamma._id, beta._id, eps))

    def tile(x, reps):  # src/nn.ts:251-253
        return Tensor(native.tile(x._id, list(reps)))

    def softmax(x, dim=-1):  # src/nn.ts:77-79
        return Tensor(native.softmaxOp(x._id, dim))

    def layerNorm(x, gamma, beta, eps=1e-5):  # src/nn.ts LayerNorm -> native.layernormOp
        return Tensor(native.layernormOp(x._id, gamma._id, beta._id, eps))

    def biasGelu(x, bias):  # src/nn.ts:153-155
        return Tensor(native.biasGelu(x._id, bias._id))

    def flashAttention(q, k, v, scale, causal=True):  # src/nn.ts:107-110
        return Tensor(native.flashAttention(q._id, k._id, v._id, scale, causal))

    class KvCache:  # src/nn.ts:111-151
        def __init__(self, batchSize, numHeads, headDim, maxSeqLen, quantized=True):
            if not hasattr(native, "kvCacheCreate"):
                raise RuntimeError("kv cache is not available in this native build")
            requested = quantized and hasattr(native, "flashAttention")
            self.cacheId = native.kvCacheCreate(batchSize, numHeads, headDim, maxSeqLen, requested)

        def decodeStep(self, q, k, v, scale):
            return Tensor(native.kvCacheDecodeStep(self.cacheId, q._id, k._id, v._id, scale))

        def append(self, k, v):
            native.kvCacheAppend(self.cacheId, k._id, v._id)

        def length(self):
            return int(native.kvCacheLen(self.cacheId))

        def isQuantized(self):
            return bool(native.kvCacheQuantized(self.cacheId))

        def reset(self):
            native.kvCacheReset(self.cacheId)

        def free(self):
            native.kvCacheFree(self.cacheId)

    class Adam:  # src/optimizer.ts:33-70: options object, defaults lr 6e-4, beta2 0.95
        def __init__(self, parameters, lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weightDecay=0.0):
            self.parameters = list(parameters)
            self.lr, self.beta1, self.beta2, self.eps, self.weightDecay = lr, beta1, beta2, eps, weightDecay
            self.t = 0

        def zeroGrad(self):
            native.zeroGrad([p.value._id for p in self.parameters])

        def step(self, maxGradNorm=0.0):
            self.t += 1
            ids = [p.value._id for p in self.parameters]
            return native.clipAndStep(ids, self.lr, self.beta1, self.beta2, self.eps, self.weightDecay, self.t, maxGradNorm)

    class GradScaler:  # src/optimizer.ts:72-121
        def __init__(self, initScale=65536.0, growthFactor=2.0, backoffFactor=0.5, growthInterval=2000):
            self.scale, self.growthFactor, self.backoffFactor = initScale, growthFactor, backoffFactor
            self.growthInterval, self.stepsSinceGrowth = growthInterval, 0

        def getScale(self):
            return self.scale

        def scaleLoss(self, loss):
            return loss.mul(self.scale)

        def unscaleAndStep(self, optimizer, maxGradNorm=0.0):
            ids = [p.value._id for p in optimizer.parameters]
            if native.scaleGrads(ids, 1.0 / self.scale):
                self.scale *= self.backoffFactor
                self.stepsSinceGrowth = 0
                optimizer.zeroGrad()
                return {"gradNorm": 0, "skipped": True}
            gradNorm = optimizer.step(maxGradNorm)
            self.stepsSinceGrowth += 1
            if self.stepsSinceGrowth >= self.growthInterval:
                self.scale *= self.growthFactor
                self.stepsSinceGrowth = 0
            return {"gradNorm": gradNorm, "skipped": False}

    return SimpleNamespace(native=native, Embedding=Embedding, crossEntropyLossGpu=crossEntropyLossGpu, dropout=dropout,
                           residualLayerNorm=residualLayerNorm, tile=tile, GradScaler=GradScaler, Tensor=Tensor, Parameter=Parameter, Module=Module, Linear=Linear, ReLU=ReLU,
                           GELU=GELU, mseLoss=mseLoss, crossEntropyLoss=crossEntropyLoss, softmax=softmax, biasGelu=biasGelu, layerNorm=layerNorm,
                           flashAttention=flashAttention, KvCache=KvCache, Adam=Adam)
