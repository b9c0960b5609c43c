"""Instruction blocks: the operator API of the reference's instructions.js.

Each `*Block.newInstance(...)` takes the reference's arguments in the reference's
order and returns `{"resultBuffer": Buffer, "passes": [...]}`; a pass is
`{"flag": "compute", "op": <C-ABI entry point>, "args": (...)}` or
`{"flag": "copy", "src", "srcOffset", "dst", "dstOffset", "size"}` and is executed
by `run_passes` (the command encoding loop of model.js:245-257), which calls the
HIP library instead of a WebGPU command encoder.
"""
import ctypes as C
import math

import numpy as np

from . import _lib


class Buffer:
    """A device buffer handle (what the reference holds as a GPUBuffer)."""

    def __init__(self, dims, handle=None):
        self.dims = tuple(int(x) for x in dims)
        self.size = 4 * int(np.prod(self.dims))
        if handle is None:
            h = C.c_uint64(0)
            _lib.call("wgpt_alloc", self.size, C.byref(h))
            handle = h.value
        self.handle = handle
        self.destroyed = False

    def destroy(self):
        if not self.destroyed:
            _lib.call("wgpt_free", self.handle)
            self.destroyed = True
            if getattr(self, "rows", None) is not None:  # row form of a transposed vocabulary chunk (DeEmbedBlock)
                self.rows.destroy()
                self.rows = None

    def upload(self, data, offset=0):
        a = np.ascontiguousarray(data)
        _lib.call("wgpt_upload", self.handle, offset, a.ctypes.data_as(C.c_void_p), a.nbytes)

    def download(self, dtype=np.float32, count=None, offset=0):
        n = self.size // np.dtype(dtype).itemsize if count is None else count
        out = np.empty(n, dtype)
        _lib.call("wgpt_download", out.ctypes.data_as(C.c_void_p), self.handle, offset, out.nbytes)
        return out


def init_tensor(data, dims, ops=("storage",)):
    """GPT.initTensor(data, dims, ops), model.js:490-500. `ops` (usage flags) is
    accepted for signature compatibility; every buffer is plain device memory."""
    buf = Buffer(dims)
    buf.upload(np.asarray(data).reshape(-1))
    return buf


def wgSize(dim, size):  # globals.js:45
    return math.ceil(dim / size)


class Block:
    """Base class, instructions.js:7-139. The pipeline and bind-group caches have
    no counterpart; the double-buffered result-buffer pool is kept: buffers made
    during one run are released by the clearBufferCache() after the next."""

    def __init__(self):
        self.name = ""
        self.device = None
        self.boundBufferCache = []
        self.unboundBufferCache = []

    def initialize(self, device):
        self.device = device
        self.boundBufferCache = []
        self.unboundBufferCache = []

    def initResultBuffer(self, dims):
        return self.initBuffer(["storage", "copy_from"], dims)

    def initBuffer(self, ops, dims, key=""):
        self.bufferSize(dims[0], dims[1] if len(dims) > 1 else 1)
        buf = Buffer(dims)
        self.boundBufferCache.append(buf)
        return buf

    def bufferSize(self, dimA, dimB=1):
        size = dimA * dimB * 4
        if size > self.device.limits["maxStorageBufferBindingSize"]:
            raise ValueError("Buffer size exceeds GPU limit.")  # instructions.js:79
        return size

    def clearBufferCache(self):
        for b in self.unboundBufferCache:
            b.destroy()
        self.unboundBufferCache = self.boundBufferCache
        self.boundBufferCache = []

    def destroyBuffers(self):
        for b in self.unboundBufferCache + self.boundBufferCache:
            b.destroy()
        self.unboundBufferCache = []
        self.boundBufferCache = []

    def destroy(self):
        self.destroyBuffers()


def _compute(op, *args):
    return {"flag": "compute", "op": op, "args": args}


class FastMatMulBlockClass(Block):
    def __init__(self):
        super().__init__()
        self.name = "fastMatMul"

    def newInstance(self, rows, cols, shared, inputBuffer, weightsBuffer, biasBuffer):
        if cols % 8 != 0:
            raise ValueError("Cols must be divisible by 16.")  # instructions.js:158
        resultBuffer = self.initResultBuffer([rows, cols])
        bias = biasBuffer.handle if biasBuffer is not None else 0
        return {"resultBuffer": resultBuffer,
                "passes": [_compute("wgpt_matmul_bias", rows, cols, shared, inputBuffer.handle, weightsBuffer.handle,
                                    bias, resultBuffer.handle)]}

    def newInt8Instance(self, rows, cols, shared, inputBuffer, packedWeightsBuffer, scaleBuffer, biasBuffer=None):
        """other/int8-gemm.js as a block: weights are packed int8 words + per-column scales."""
        if cols % 8 != 0:
            raise ValueError("Cols must be divisible by 16.")
        resultBuffer = self.initResultBuffer([rows, cols])
        bias = biasBuffer.handle if biasBuffer is not None else 0
        return {"resultBuffer": resultBuffer,
                "passes": [_compute("wgpt_matmul_bias_i8", rows, cols, shared, inputBuffer.handle,
                                    packedWeightsBuffer.handle, scaleBuffer.handle, bias, resultBuffer.handle)]}


class ResidualBlockClass(Block):
    def __init__(self):
        super().__init__()
        self.name = "residual"

    def newInstance(self, rows, cols, outputBuf, residualBuf):
        if cols % 4 != 0:
            raise ValueError("Cols must be divisible by 4.")  # instructions.js:337
        resultBuffer = self.initResultBuffer([rows, cols])
        return {"resultBuffer": resultBuffer,
                "passes": [_compute("wgpt_residual", rows, cols, outputBuf.handle, residualBuf.handle, resultBuffer.handle)]}


class LayerNormBlockClass(Block):
    def __init__(self):
        super().__init__()
        self.name = "layerNorm"

    def newInstance(self, rows, cols, inputBuffer, gammaBuffer, betaBuffer):
        if cols % 4 != 0:
            raise ValueError("Cols must be divisible by 4.")  # instructions.js:410
        resultBuffer = self.initResultBuffer([rows, cols])
        return {"resultBuffer": resultBuffer,
                "passes": [_compute("wgpt_layernorm", rows, cols, inputBuffer.handle, gammaBuffer.handle,
                                    betaBuffer.handle, resultBuffer.handle)]}


class SoftmaxBlockClass(Block):
    def __init__(self):
        super().__init__()
        self.name = "softmax"

    def newInstance(self, rows, cols, inputBuffer, transpose=False):
        # transpose: the same values stored as [cols, rows] (instructions.js:594)
        resultBuffer = self.initResultBuffer([cols, rows] if transpose else [rows, cols])
        return {"resultBuffer": resultBuffer,
                "passes": [_compute("wgpt_softmax_t" if transpose else "wgpt_softmax", rows, cols, inputBuffer.handle,
                                    resultBuffer.handle)]}


class GeluBlockClass(Block):
    def __init__(self):
        super().__init__()
        self.name = "gelu"

    def newInstance(self, rows, cols, inputBuf):
        if cols % 4 != 0:
            raise ValueError("Cols must be divisible by 4.")  # instructions.js:684
        resultBuffer = self.initResultBuffer([rows, cols])
        return {"resultBuffer": resultBuffer,
                "passes": [_compute("wgpt_gelu", rows, cols, inputBuf.handle, resultBuffer.handle)]}


class EmbedBlockClass(Block):
    def __init__(self):
        super().__init__()
        self.name = "embed"

    def newInstance(self, idx, seq_length, n_embd, vocab_chunk_size, embdBuffers, posEmbdBuffer, ResidualBlock):
        """instructions.js:790-827. `embdBuffers` is either the single un-chunked [V, d] table (one fused
        gather + add) or the reference's list of zero-padded [vocab_chunk_size, d] chunks (model.js:348-361):
        then token i is row idx[i] % vocab_chunk_size of chunk floor(idx[i] / vocab_chunk_size), copied row by
        row, and the positional rows are added by the ResidualBlock, as the reference does (795-821)."""
        ids = np.ascontiguousarray(idx, dtype=np.int32)
        if len(embdBuffers) == 1:
            resultBuffer = self.initResultBuffer([seq_length, n_embd])
            V = embdBuffers[0].dims[0]
            return {"resultBuffer": resultBuffer,
                    "passes": [_compute("wgpt_embed", ids.ctypes.data_as(C.POINTER(C.c_int32)), seq_length, n_embd, V,
                                        embdBuffers[0].handle, posEmbdBuffer.handle, resultBuffer.handle)],
                    "_keepalive": ids}
        row = 4 * n_embd
        embdOutputBuffer = self.initBuffer(["storage", "copy_to"], [seq_length, n_embd])
        posEmbdOutputBuffer = self.initBuffer(["storage", "copy_to"], [seq_length, n_embd])
        passes = []
        for i in range(seq_length):
            chunk, within = divmod(int(ids[i]), vocab_chunk_size)
            if int(ids[i]) < 0 or chunk >= len(embdBuffers):
                raise ValueError("token id outside the embedding chunks")
            passes.append({"flag": "copy", "src": embdBuffers[chunk], "srcOffset": row * within,
                           "dst": embdOutputBuffer, "dstOffset": row * i, "size": row})
        passes.append({"flag": "copy", "src": posEmbdBuffer, "srcOffset": 0, "dst": posEmbdOutputBuffer, "dstOffset": 0,
                       "size": row * seq_length})
        res = (ResidualBlock or globals()["ResidualBlock"]).newInstance(seq_length, n_embd, embdOutputBuffer, posEmbdOutputBuffer)
        return {"resultBuffer": res["resultBuffer"], "passes": passes + res["passes"]}


class DeEmbedBlockClass(Block):
    def __init__(self):
        super().__init__()
        self.name = "deembed"

    def newInstance(self, n_embd, vocab_size, padded_vocab_size, seq_length, vocab_chunk_size, embedBuffer, deEmbeddingsBuffers):
        """instructions.js:844-888. `deEmbeddingsBuffers` is either the single [V, d] table (no host-side
        transposes, no chunk copies) or the reference's list of transposed, zero-padded [d, vocab_chunk_size]
        chunks (model.js:362-363). A chunk is turned back into rows on the device the first time it is seen
        (wgpt_transpose; the row form is kept with the buffer, which the reference also makes once, at load), and
        every chunk's logits go to their offset in the result, the last copy dropping the padding columns
        (instructions.js:873-880). The products are the single-table kernel's, row by row: same logits bit for bit."""
        resultBuffer = self.initBuffer(["map_read", "copy_to"], [vocab_size])
        if len(deEmbeddingsBuffers) == 1 and deEmbeddingsBuffers[0].dims[0] == vocab_size:
            return {"resultBuffer": resultBuffer,
                    "passes": [_compute("wgpt_deembed", n_embd, vocab_size, seq_length, embedBuffer.handle,
                                        deEmbeddingsBuffers[0].handle, resultBuffer.handle)]}
        passes = []
        for i, chunkBuffer in enumerate(deEmbeddingsBuffers):
            if tuple(chunkBuffer.dims) != (n_embd, vocab_chunk_size):
                raise ValueError("a de-embedding chunk must be [n_embd, vocab_chunk_size]")
            if getattr(chunkBuffer, "rows", None) is None:
                chunkBuffer.rows = Buffer([vocab_chunk_size, n_embd])
                _lib.call("wgpt_transpose", n_embd, vocab_chunk_size, chunkBuffer.handle, chunkBuffer.rows.handle)
            valid = min(vocab_chunk_size, vocab_size - i * vocab_chunk_size)
            if valid <= 0:
                break
            chunkResultBuffer = self.initResultBuffer([valid])
            passes.append(_compute("wgpt_deembed", n_embd, valid, seq_length, embedBuffer.handle, chunkBuffer.rows.handle,
                                   chunkResultBuffer.handle))
            passes.append({"flag": "copy", "src": chunkResultBuffer, "srcOffset": 0, "dst": resultBuffer,
                           "dstOffset": 4 * i * vocab_chunk_size, "size": 4 * valid})
        return {"resultBuffer": resultBuffer, "passes": passes}


class AttentionBlockClass(Block):
    def __init__(self):
        super().__init__()
        self.name = "attention"

    def newFusedInstance(self, seq_length, n_embd, attentionDotProductScale, n_head, head_size, inputBuffer,
                         qWeightsBuffer, qBiasBuffer, kWeightsBuffer, kBiasBuffer, vWeightsBuffer, vBiasBuffer,
                         linearWeightsBuffer, linearBiasBuffer, FastMatMulBlock=None, SoftmaxBlock=None):
        """instructions.js:985-1099: one fused launch sequence instead of eight passes."""
        resultBuffer = self.initResultBuffer([seq_length, n_embd])
        hs = [b.handle for b in (inputBuffer, qWeightsBuffer, qBiasBuffer, kWeightsBuffer, kBiasBuffer, vWeightsBuffer,
                                 vBiasBuffer, linearWeightsBuffer, linearBiasBuffer)]
        return {"resultBuffer": resultBuffer,
                "passes": [_compute("wgpt_attention", seq_length, n_embd, C.c_float(attentionDotProductScale), n_head,
                                    head_size, *hs, resultBuffer.handle)]}


FastMatMulBlock = FastMatMulBlockClass()
AttentionBlock = AttentionBlockClass()
ResidualBlock = ResidualBlockClass()
EmbedBlock = EmbedBlockClass()
DeEmbedBlock = DeEmbedBlockClass()
GeluBlock = GeluBlockClass()
LayerNormBlock = LayerNormBlockClass()
SoftmaxBlock = SoftmaxBlockClass()

# globals.js:11
operations = [FastMatMulBlock, AttentionBlock, ResidualBlock, EmbedBlock, DeEmbedBlock, GeluBlock, LayerNormBlock, SoftmaxBlock]


def initializeOperations(device):  # globals.js:13-15
    for op in operations:
        op.initialize(device)


def destroyOperationBuffers():  # globals.js:17-19
    for op in operations:
        op.destroyBuffers()


def clearOperationCache():  # globals.js:21-23
    for op in operations:
        op.clearBufferCache()


def destroyOperations():  # globals.js:25-27
    for op in operations:
        op.destroy()


def run_passes(passes):
    """The command-encoding loop of model.js:245-257 over the HIP library."""
    for p in passes:
        if p["flag"] == "compute":
            _lib.call(p["op"], *p["args"])
        elif p["flag"] == "copy":
            _lib.call("wgpt_copy", p["dst"].handle, p["dstOffset"], p["src"].handle, p["srcOffset"], p["size"])
        else:
            raise ValueError(f"unknown pass flag {p['flag']!r}")


class Device:
    """Stands in for the GPUDevice the reference threads through its blocks: it owns
    the library's lifetime and reports the limits the reference checks against."""

    def __init__(self, index=0):
        _lib.init(index)
        name = C.create_string_buffer(128)
        cus = C.c_int(0)
        hbm = C.c_uint64(0)
        _lib.call("wgpt_device_info", name, 128, C.byref(cus), C.byref(hbm))
        self.name = name.value.decode()
        self.compute_units = cus.value
        self.hbm_bytes = hbm.value
        # No binding-size limit exists here; the whole of HBM is addressable from a kernel.
        self.limits = {"maxStorageBufferBindingSize": hbm.value, "maxBufferSize": hbm.value}

    def sync(self):
        _lib.call("wgpt_sync")

    def destroy(self):
        _lib.shutdown()
