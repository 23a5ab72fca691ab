"""The .one model file: a writer that lays a graph out the way the reference converter does
(tools/onnx2one/onnx2one.cpp:1294-1355) and a reader that walks it the way the reference host does
(host/net.h:138-221).

    [ONE_MODEL_DESC_S][node configs][initialisers][io configs]        every piece padded to 64 bytes
      node config   the operator's *_CONFIG_S, BASE_CONFIG_S first, op_type selects the struct
      initialiser   OPERAND_S, then the raw data
      io config     IO_CONFIG_S with op_type "io" and op_name "input" / "output"

The converter itself needs protobuf and an ONNX file; `OneModel` builds the same bytes from Python calls, one per
node, for the operator set of this package (Conv, MatMul, Gemm, Add, Relu, MaxPool, GlobalAveragePool, Gelu,
LayerNormalization, Softmax, Transpose, Flatten, Reshape).
"""
import ctypes as C

import numpy as np

from . import abi

CFG_TYPES = {
    "Conv": abi.CONV_CONFIG_S, "MatMul": abi.MATMUL_CONFIG_S, "Gemm": abi.GEMM_CONFIG_S, "Add": abi.PLAIN_CONFIG_S,
    "Relu": abi.PLAIN_CONFIG_S, "GlobalAveragePool": abi.PLAIN_CONFIG_S, "Gelu": abi.PLAIN_CONFIG_S,
    "MaxPool": abi.MAX_POOL_CONFIG_S, "LayerNormalization": abi.LAYERNORMALIZATION_CONFIG_S,
    "Softmax": abi.SOFTMAX_CONFIG_S, "Transpose": abi.TRANSPOSE_CONFIG_S, "Flatten": abi.FLATTEN_CONFIG_S,
    "Reshape": abi.RESHAPE_CONFIG_S,
    # activation nodes of a file that has not been through the offline optimiser (tools/optimize/op_fusion.hpp:75-192)
    "Clip": abi.CLIP_CONFIG_S, "LeakyRelu": abi.LEAKYRELU_CONFIG_S, "HardSigmoid": abi.HARD_SIGMOID_CONFIG_S,
    "Sigmoid": abi.PLAIN_CONFIG_S, "Mul": abi.PLAIN_CONFIG_S,
}
# ONNX element type numbers (common/nn_common.h:92-110)
DTYPES = {abi.TYPE_FP32: np.float32, abi.TYPE_INT8: np.int8, abi.TYPE_INT32: np.int32, 7: np.int64}
TYPE_OF = {np.dtype(v): k for k, v in DTYPES.items()}


def align64(n):
    """common/utils_c.h:4-7"""
    return (n + 63) & ~63


def _operand(name, shape, dtype=abi.TYPE_FP32, fixed=False):
    o = abi.OPERAND_S()
    o.operand_name = name.encode()
    o.is_fixed_val = int(fixed)
    o.dim_num_of_shapes = max(1, len(shape)) if fixed else len(shape)   # a scalar initialiser counts one dimension
    for i in range(abi.SHAPE_LEN):
        o.shapes[i] = int(shape[i]) if i < len(shape) else 1
    o.data_type = dtype
    return o


class OneModel:
    """Collects inputs, outputs, initialisers and nodes; tobytes() gives the file."""

    def __init__(self):
        self.ios = []        # (kind, name, shape)
        self.inits = []      # (name, array)
        self.nodes = []      # config structs

    # ---- graph pieces ----------------------------------------------------------------------------------
    def input(self, name, shape):
        self.ios.append(("input", name, tuple(shape)))
        return name

    def output(self, name, shape):
        self.ios.append(("output", name, tuple(shape)))
        return name

    def init(self, name, array):
        a = np.ascontiguousarray(array)
        if a.dtype not in TYPE_OF:
            raise ValueError(f"initialiser {name}: dtype {a.dtype} has no .one element type here")
        self.inits.append((name, a))
        return name

    def node(self, op_type, name, ins, outs, **fields):
        cfg = CFG_TYPES[op_type]()
        b = cfg.op_base_cfg
        b.op_type, b.op_name = op_type.encode(), name.encode()
        for i, n in enumerate(ins):
            b.in_operand_name[i].value = n.encode()
        for i, n in enumerate(outs):
            b.out_operand_name[i].value = n.encode()
        b.in_operand_num, b.out_operand_num = len(ins), len(outs)
        for k, v in fields.items():
            field = getattr(cfg, k)
            if isinstance(field, C.Array):
                for i, x in enumerate(v):
                    field[i] = x
            else:
                setattr(cfg, k, v)
        self.nodes.append(cfg)
        return outs[0]

    # ---- operators -------------------------------------------------------------------------------------
    def conv(self, name, x, weight, bias, out, stride=1, pad=0, group=1, act=abi.NOT_ACT, clip=(0.0, 0.0), quant=None, leaky=0.0,
             hard=(0.0, 0.0)):
        """weight [cout, cin/group, kh, kw] fp32 and bias [cout] (or None) become initialisers name.weight / name.bias.
        quant=(weight_aux [cout], input_scale) marks the W8A32 form the offline quantiser writes
        (tools/optimize/model_quant.hpp:14-25, :655-670): weight is then int8 and bias int32, both stored at the
        front of initialisers that keep their fp32 size and type."""
        pads = (pad,) * 4 if isinstance(pad, int) else tuple(pad)
        strides = (stride, stride) if isinstance(stride, int) else tuple(stride)
        fields = {}
        if quant is None:
            w = np.asarray(weight, dtype=np.float32)
            b = None if bias is None else np.asarray(bias, dtype=np.float32)
        else:
            aux, input_scale = quant
            w8 = np.ascontiguousarray(weight, dtype=np.int8)
            w = np.zeros(w8.shape, dtype=np.float32)
            w.reshape(-1).view(np.int8)[:w8.size] = w8.reshape(-1)
            b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32).view(np.float32)
            fields = dict(ifmap_quant2=abi.TYPE_INT8, input_scale=float(input_scale),
                          weight_aux=tuple(float(v) for v in np.asarray(aux, dtype=np.float32)))
        ins = [x, self.init(name + ".weight", w)]
        if b is not None:
            ins.append(self.init(name + ".bias", b))
        return self.node("Conv", name, ins, [out], has_bias=int(b is not None), dilations=(1, 1), group=group,
                         kernel_shape=w.shape[2:], pads=pads, strides=strides, act_type=act, clip_min=clip[0],
                         clip_max=clip[1], leaky_relu_alpha=leaky, hard_sigmoid_alpha=hard[0], hard_sigmoid_beta=hard[1], **fields)

    def gemm(self, name, x, weight, bias, out):
        """out = x @ weight[N, K]^T + bias (device/x86/Gemm/gemm.c)"""
        ins = [x, self.init(name + ".weight", np.asarray(weight, dtype=np.float32)),
               self.init(name + ".bias", np.asarray(bias, dtype=np.float32))]
        return self.node("Gemm", name, ins, [out], has_bias=1, alpha=1.0, beta=1.0, transB=1)

    def matmul(self, name, a, b, out):
        """b: the name of an operand, or an array [K, N] that becomes an initialiser"""
        if not isinstance(b, str):
            b = self.init(name + ".weight", np.asarray(b, dtype=np.float32))
        return self.node("MatMul", name, [a, b], [out])

    def add(self, name, a, b, out):
        """b: the name of an operand, or an array that becomes an initialiser"""
        if not isinstance(b, str):
            b = self.init(name + ".b", np.asarray(b, dtype=np.float32))
        return self.node("Add", name, [a, b], [out])

    def relu(self, name, x, out):
        return self.node("Relu", name, [x], [out])

    def clip(self, name, x, out, lo, hi):
        return self.node("Clip", name, [x], [out], min=lo, max=hi)

    def leaky_relu(self, name, x, out, alpha):
        return self.node("LeakyRelu", name, [x], [out], alpha=alpha)

    def sigmoid(self, name, x, out):
        return self.node("Sigmoid", name, [x], [out])

    def hard_sigmoid(self, name, x, out, alpha, beta):
        return self.node("HardSigmoid", name, [x], [out], alpha=alpha, beta=beta)

    def mul(self, name, a, b, out):
        return self.node("Mul", name, [a, b], [out])

    def gelu(self, name, x, out):
        return self.node("Gelu", name, [x], [out])

    def maxpool(self, name, x, out, kernel, stride, pad):
        return self.node("MaxPool", name, [x], [out], kernel_shape=(kernel, kernel), pads=(pad,) * 4,
                         strides=(stride, stride))

    def global_avgpool(self, name, x, out):
        return self.node("GlobalAveragePool", name, [x], [out])

    def layernorm(self, name, x, weight, bias, out, axis=-1):
        ins = [x, self.init(name + ".weight", np.asarray(weight, dtype=np.float32)),
               self.init(name + ".bias", np.asarray(bias, dtype=np.float32))]
        return self.node("LayerNormalization", name, ins, [out], axes=(axis,), axes_num=1)

    def softmax(self, name, x, out, axis=-1):
        return self.node("Softmax", name, [x], [out], axis=axis)

    def transpose(self, name, x, out, perm):
        return self.node("Transpose", name, [x], [out], perm=tuple(perm), perm_num=len(perm))

    def flatten(self, name, x, out, axis=1):
        return self.node("Flatten", name, [x], [out], axis=axis)

    def reshape(self, name, x, out, shape):
        return self.node("Reshape", name, [x], [out], dst_shape=tuple(shape), dst_shape_num=len(shape))

    # ---- layout ----------------------------------------------------------------------------------------
    def _fill_producers_consumers(self):
        """tools/onnx2one/onnx2one.cpp:1117-1227: per node, who makes its non-initialiser inputs and who reads
        its outputs; an io node appears as type "io" with the operand's name"""
        producers, consumers = {}, {}
        for cfg in self.nodes:
            b = cfg.op_base_cfg
            me = (b.op_type, b.op_name)
            for i in range(b.in_operand_num):
                lst = consumers.setdefault(b.in_operand_name[i].value, [])
                if me not in lst:
                    lst.append(me)
            for i in range(b.out_operand_num):
                lst = producers.setdefault(b.out_operand_name[i].value, [])
                if me not in lst:
                    lst.append(me)
        for kind, name, _ in self.ios:
            (producers if kind == "input" else consumers).setdefault(name.encode(), []).append((b"io", name.encode()))
        init_names = {n.encode() for n, _ in self.inits}
        for cfg in self.nodes:
            b = cfg.op_base_cfg
            b.producer_num = b.consumer_num = 0
            for i in range(b.in_operand_num):
                key = b.in_operand_name[i].value
                if key in init_names:
                    continue
                for t, n in producers.get(key, []):
                    if b.producer_num < abi.OPERAND_MAXNUM:
                        b.producer[b.producer_num].op_type, b.producer[b.producer_num].op_name = t, n
                        b.producer_num += 1
            for i in range(b.out_operand_num):
                for t, n in consumers.get(b.out_operand_name[i].value, []):
                    if b.consumer_num < abi.OPERAND_MAXNUM:
                        b.consumer[b.consumer_num].op_type, b.consumer[b.consumer_num].op_name = t, n
                        b.consumer_num += 1

    def tobytes(self):
        self._fill_producers_consumers()
        head = align64(C.sizeof(abi.ONE_MODEL_DESC_S))
        cfg_bytes = sum(align64(C.sizeof(c)) for c in self.nodes)
        init_bytes = sum(align64(C.sizeof(abi.OPERAND_S) + a.nbytes) for _, a in self.inits)
        io_bytes = len(self.ios) * align64(C.sizeof(abi.IO_CONFIG_S))
        buf = bytearray(head + cfg_bytes + init_bytes + io_bytes)
        h = abi.ONE_MODEL_DESC_S.from_buffer(buf)
        h.one_model_magic_num = abi.ONE_MAGIC_NUM
        h.node_cnt, h.node_cfg_offset = len(self.nodes), head
        h.init_cnt, h.init_info_offset = len(self.inits), head + cfg_bytes
        h.io_cfg_cnt, h.io_cfg_offset = len(self.ios), head + cfg_bytes + init_bytes
        # defaults of the converter: 512 MB shared scratch, x86 tiles 32/1024/8, device tiles 16 (onnx2one.cpp:1332-1350)
        h.useful_info.public_buf_info.public_buf_size = 512 * 1024 * 1024
        bi = h.useful_info.block_info
        bi.x86_gemm_single_threads_tile_m, bi.x86_gemm_single_threads_tile_n, bi.x86_gemm_single_threads_tile_k = 32, 1024, 8
        bi.x86_gemm_multi_threads_tile_m, bi.x86_gemm_multi_threads_tile_n, bi.x86_gemm_multi_threads_tile_k = 32, 1024, 8
        bi.cuda_gemm_tile_m = bi.cuda_gemm_tile_n = bi.cuda_gemm_tile_k = 16
        del h, bi
        off = head
        for c in self.nodes:
            buf[off:off + C.sizeof(c)] = bytes(c)
            off += align64(C.sizeof(c))
        for name, a in self.inits:
            o = _operand(name, a.shape, TYPE_OF[a.dtype], fixed=True)
            buf[off:off + C.sizeof(o)] = bytes(o)
            buf[off + C.sizeof(o):off + C.sizeof(o) + a.nbytes] = a.tobytes()
            off += align64(C.sizeof(o) + a.nbytes)
        for kind, name, shape in self.ios:
            io = abi.IO_CONFIG_S()
            io.op_type, io.op_name = b"io", kind.encode()
            io.operand = _operand(name, shape)
            buf[off:off + C.sizeof(io)] = bytes(io)
            off += align64(C.sizeof(io))
        return bytes(buf)


def parse(data):
    """Walks a .one file like host/net.h:138-221.  Returns a dict: header, nodes [(type, config struct)],
    inits {name: array}, inputs / outputs [(name, shape)]."""
    data = bytes(data)
    h = abi.ONE_MODEL_DESC_S.from_buffer_copy(data[:C.sizeof(abi.ONE_MODEL_DESC_S)])
    if h.one_model_magic_num != abi.ONE_MAGIC_NUM:
        raise ValueError("not a .one file")
    nodes, off = [], h.node_cfg_offset
    for _ in range(h.node_cnt):
        op_type = data[off:off + abi.NAME_LEN].split(b"\0", 1)[0].decode()
        if op_type not in CFG_TYPES:
            raise ValueError(f"node type {op_type} is outside this package's operator set")
        cls = CFG_TYPES[op_type]
        nodes.append((op_type, cls.from_buffer_copy(data[off:off + C.sizeof(cls)])))
        off += align64(C.sizeof(cls))
    inits, off = {}, h.init_info_offset
    for _ in range(h.init_cnt):
        o = abi.OPERAND_S.from_buffer_copy(data[off:off + C.sizeof(abi.OPERAND_S)])
        dtype = np.dtype(DTYPES[o.data_type])
        n = int(np.prod([o.shapes[i] for i in range(abi.SHAPE_LEN)]))
        start = off + C.sizeof(abi.OPERAND_S)
        shape = tuple(o.shapes[i] for i in range(o.dim_num_of_shapes))
        inits[o.operand_name.decode()] = np.frombuffer(data, dtype=dtype, count=n, offset=start).reshape(shape)
        off += align64(C.sizeof(abi.OPERAND_S) + n * dtype.itemsize)
    inputs, outputs, off = [], [], h.io_cfg_offset
    for _ in range(h.io_cfg_cnt):
        io = abi.IO_CONFIG_S.from_buffer_copy(data[off:off + C.sizeof(abi.IO_CONFIG_S)])
        shape = tuple(io.operand.shapes[i] for i in range(io.operand.dim_num_of_shapes))
        (inputs if io.op_name == b"input" else outputs).append((io.operand.operand_name.decode(), shape))
        off += align64(C.sizeof(abi.IO_CONFIG_S))
    return {"header": h, "nodes": nodes, "inits": inits, "inputs": inputs, "outputs": outputs}
