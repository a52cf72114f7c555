"""Python view of libmi355_strix.so (include/mi355_strix.h) for tests and the benchmark.

torch is used for device memory and streams only; every computation goes through the C ABI. There is no CPU or
eager fallback: a missing library or a missing GPU raises."""
import ctypes as C
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmi355_strix.so")

TYPE_Q5_1, TYPE_Q8_0, TYPE_Q4_K, TYPE_Q5_K, TYPE_Q6_K = 7, 8, 12, 13, 14
INPUT_F32, INPUT_F16, INPUT_BF16 = 0, 1, 2
LOGITS_FMA, LOGITS_LANE32 = 0, 1
COMBINE_FMA_SLOT, COMBINE_MULADD_ASC, COMBINE_NONE, COMBINE_BF16_STEPS = 0, 1, 2, 3
EXP_GFX1151, EXP_DECLARED, EXP_LIBM = 0, 1, 2
STATUS_INVALID_ROUTE, STATUS_NONFINITE_ACTIVATION, STATUS_INVALID_DELTA, STATUS_NONFINITE_PROJECTION, STATUS_AGGREGATE = 1, 2, 4, 8, 16
E_INVALID_ARGUMENT, E_UNSUPPORTED, E_HIP = -1, -2, -3
Q8_0_BLOCK, Q4_K_BLOCK = 34, 144
UNION_MAX_ROWS, UNION_MAX_TOP_K, UNION_PLAN_BYTES = 8, 16, 1552      # expert-union plan of a verify window (mi355_a8_*_union)


class StrixError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"mi355_strix error {code}: {message}")
        self.code = code


class Q8a8View(C.Structure):
    _fields_ = [("weight", C.c_void_p), ("codes", C.c_void_p), ("deltas", C.c_void_p), ("out", C.c_void_p),
                ("row_bytes", C.c_uint32), ("in_", C.c_uint32), ("count", C.c_uint32), ("rows", C.c_uint32),
                ("x_stride", C.c_uint32), ("out_stride", C.c_uint32), ("accumulate", C.c_uint32)]


class RoutePolicy(C.Structure):
    _fields_ = [("experts", C.c_uint32), ("top_k", C.c_uint32), ("logits_order", C.c_uint32),
                ("renorm_eps", C.c_float), ("scale", C.c_float), ("renormalize", C.c_uint32),
                ("renorm_single", C.c_uint32), ("exp_kind", C.c_uint32), ("shared_experts", C.c_uint32),
                ("shared_slot_weights", C.c_void_p)]


class MoeWeights(C.Structure):
    _fields_ = [("hidden", C.c_uint32), ("ffn", C.c_uint32), ("experts", C.c_uint32), ("top_k", C.c_uint32),
                ("gate_type", C.c_uint32), ("down_type", C.c_uint32),
                ("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p),
                ("gate_expert_stride", C.c_uint64), ("gate_row_stride", C.c_uint64),
                ("down_expert_stride", C.c_uint64), ("down_row_stride", C.c_uint64), ("exp_kind", C.c_uint32),
                ("swiglu_limit", C.c_float)]


class MoeRows(C.Structure):
    _fields_ = [("input", C.c_void_p), ("input_kind", C.c_uint32), ("input_stride", C.c_uint64),
                ("routes", C.c_void_p), ("route_weights", C.c_void_p),
                ("codes", C.c_void_p), ("deltas", C.c_void_p), ("sums", C.c_void_p), ("status", C.c_void_p),
                ("gate_out", C.c_void_p), ("up_out", C.c_void_p), ("h_out", C.c_void_p),
                ("down_codes", C.c_void_p), ("down_deltas", C.c_void_p), ("down_sums", C.c_void_p),
                ("rawdots", C.c_void_p), ("base", C.c_void_p), ("output", C.c_void_p), ("output_stride", C.c_uint64),
                ("plan", C.c_void_p), ("job_status", C.c_void_p), ("h_f16", C.c_void_p)]


class DeviceBytes(C.Structure):
    _fields_ = [("address", C.c_size_t), ("bytes", C.c_uint64)]


class A8Shape(C.Structure):
    _fields_ = [("hidden", C.c_uint32), ("rows", C.c_uint32), ("experts", C.c_uint32), ("top_k", C.c_uint32), ("logical_rows", C.c_uint32)]


class A8Request(C.Structure):
    _fields_ = [("enabled", C.c_uint32), ("approved_numerical_identity", C.c_char_p), ("input", C.c_uint32), ("shape", A8Shape),
                ("gate_type", C.c_uint32), ("up_type", C.c_uint32), ("fused_gate_up", C.c_uint32), ("swiglu_limit", C.c_float)]


class A8Bindings(C.Structure):
    _fields_ = [(n, DeviceBytes) for n in ("input", "gate", "up", "routes", "codes", "deltas", "sums", "status", "output")]


class A8DownShape(C.Structure):
    _fields_ = [("hidden", C.c_uint32), ("intermediate", C.c_uint32), ("experts", C.c_uint32), ("top_k", C.c_uint32)]


class A8DownRequest(C.Structure):
    _fields_ = [("enabled", C.c_uint32), ("approved_numerical_identity", C.c_char_p), ("shape", A8DownShape), ("weight_type", C.c_uint32),
                ("swiglu_limit", C.c_float)]


class A8DownBindings(C.Structure):
    _fields_ = [(n, DeviceBytes) for n in ("intermediates", "weights", "routes", "codes", "deltas", "sums", "rawdots", "status", "aggregate_status")]


class SlotMergeTail(C.Structure):
    _fields_ = [("tickets", C.c_void_p), ("route_weights", C.c_void_p), ("accumulation", C.c_void_p), ("output", C.c_void_p),
                ("output_bf16", C.c_uint32), ("bf16_commit", C.c_uint32), ("record", C.c_void_p), ("domain", C.c_uint32)]


class Strided(C.Structure):
    _fields_ = [("base", C.c_void_p), ("stride", C.c_uint64)]


class MoeRowsStrided(C.Structure):
    _fields_ = [(n, Strided) for n in ("input", "routes", "route_weights", "codes", "deltas", "sums", "status", "intermediates", "accumulation",
                                        "down_codes", "down_deltas", "down_sums", "rawdots", "output")] + \
               [("plan", C.c_void_p), ("job_status", C.c_void_p), ("input_kind", C.c_uint32), ("output_kind", C.c_uint32)]


class PrefillRows(C.Structure):
    """mi355_prefill_rows: the strided views of the fp16 prefill (known_rows::PrefillRows, include/strix/hip_moe_q4k_a8_known_rows.hpp:75-95)."""
    _fields_ = [(n, Strided) for n in ("input", "routes", "route_weights", "status", "clear", "rawdots")] + \
               [("plan", C.c_void_p), ("job_status", C.c_void_p), ("h_f16", C.c_void_p), ("rawdots_bf16", C.c_uint32)]


class RowA8(C.Structure):
    _fields_ = [("codes", C.c_void_p), ("deltas", C.c_void_p), ("sums", C.c_void_p)]


class ExpertAssignment(C.Structure):
    _fields_ = [("row", C.c_uint32), ("slot", C.c_uint32), ("expert", C.c_uint32)]


class LayerWeights(C.Structure):
    _fields_ = [("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p), ("gate_format", C.c_uint32), ("down_format", C.c_uint32),
                ("hidden", C.c_uint32), ("ffn", C.c_uint32)]


class ExpertJob(C.Structure):
    _fields_ = [("weights", LayerWeights), ("rows", C.c_void_p), ("assignments", C.c_void_p), ("count", C.c_uint32), ("rawdots", C.c_void_p),
                ("rawdot_row_stride", C.c_uint64), ("status", C.c_void_p)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("n_dims", C.c_uint32), ("dims", C.c_uint64 * 4), ("ggml_type", C.c_uint32), ("offset", C.c_uint64),
                ("bytes", C.c_uint64)]


class GgufMoeLayerMap(C.Structure):
    _fields_ = [(n, GgufTensor) for n in ("gate", "up", "down", "router", "norm", "router_bias", "shared_gate", "shared_up", "shared_down",
                                           "shared_router")] + \
               [(n, C.c_uint32) for n in ("hidden", "ffn", "experts", "shared_ffn", "gate_type", "down_type")]


class GgufFile:
    """A parsed GGUF v3 file (strix::gguf::FileInfo, include/strix/gguf_reader.hpp:89-104): the tensor index, the metadata and the
    map of a MoE layer. Raises StrixError with the reader's reason for a file it does not admit."""

    def __init__(self, path):
        self.path = path
        self.handle = lib().mi355_gguf_open(os.fsencode(path))
        if not self.handle:
            raise StrixError(E_INVALID_ARGUMENT, lib().mi355_last_error().decode())
        self.alignment = lib().mi355_gguf_alignment(self.handle)
        self.data_offset = lib().mi355_gguf_data_offset(self.handle)

    def close(self):
        if self.handle:
            lib().mi355_gguf_close(self.handle)
            self.handle = None

    def __del__(self):
        self.close()

    @staticmethod
    def _info(t):
        return {"name": t.name.decode(), "dims": [int(t.dims[i]) for i in range(t.n_dims)], "type": int(t.ggml_type), "offset": int(t.offset),
                "bytes": int(t.bytes)}

    def tensors(self):
        out = []
        for i in range(lib().mi355_gguf_tensor_count(self.handle)):
            t = GgufTensor()
            check(lib().mi355_gguf_tensor_at(self.handle, i, C.byref(t)))
            out.append(self._info(t))
        return out

    def metadata(self, key):
        kind, u, i, f, text = C.c_uint32(), C.c_uint64(), C.c_int64(), C.c_double(), C.c_char_p()
        check(lib().mi355_gguf_metadata(self.handle, key.encode(), C.byref(kind), C.byref(u), C.byref(i), C.byref(f), C.byref(text)))
        return [u.value, i.value, f.value, text.value.decode() if text.value is not None else None, u.value][kind.value]

    def moe_layer_map(self, layer):
        m = GgufMoeLayerMap()
        check(lib().mi355_gguf_moe_layer(self.handle, layer, C.byref(m)))
        return m

    def read(self, t, device=None):
        """The bytes of a tensor (a GgufTensor of this file) as a uint8 tensor, memory-mapped from the file and uploaded when a
        device is given."""
        import numpy as np
        raw = np.memmap(self.path, dtype=np.uint8, mode="r", offset=int(t.offset), shape=(int(t.bytes),))
        host = torch.from_numpy(np.array(raw))
        return host.to(device) if device is not None else host

    def load_moe_layer(self, layer, top_k, max_rows, device="cuda", **layer_options):
        """One MoE layer of the file on the device: (MoeLayer, router weight fp32 [experts][hidden], norm weight or None, map)."""
        m = self.moe_layer_map(layer)
        gate, up, down = (self.read(t, device) for t in (m.gate, m.up, m.down))
        router = self.read(m.router, device).view(torch.float32).reshape(m.experts, m.hidden)
        norm = self.read(m.norm, device).view(torch.float32) if m.norm.bytes else None
        moe = MoeLayer(m.hidden, m.ffn, m.experts, top_k, gate, up, down, max_rows, gate_type=m.gate_type, down_type=m.down_type, **layer_options)
        return moe, router, norm, m


def device_bytes(t):
    """DeviceBytes of a tensor (None: the empty view)."""
    return DeviceBytes(0, 0) if t is None else DeviceBytes(t.data_ptr(), t.numel() * t.element_size())


_lib = None


def lib():
    """The HIP library. Raises when it was not built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        L = C.CDLL(LIB_PATH)
        L.mi355_last_error.restype = C.c_char_p
        L.mi355_version.restype = C.c_char_p
        # every pointer parameter is declared: an undeclared Python integer would be passed as a 32-bit C int
        P, U = C.c_void_p, C.c_uint32
        for name in ("prologue", "csr", "project", "down", "merge"):
            getattr(L, "mi355_moe_strided_enqueue_" + name).argtypes = [P, P, U] + ([U] if name == "prologue" else []) + [P]
        L.mi355_moe_strided_enqueue_commit.argtypes = [P, P, U, P, U, P]
        L.mi355_moe_strided_enqueue.argtypes = [P, P, U, U, P, U, P]
        L.mi355_a8_validate.argtypes = [P, P]
        L.mi355_a8_validate_down.argtypes = [P, P, U]
        L.mi355_a8_enqueue_probe.argtypes = [P, P, P]
        L.mi355_a8_enqueue_down_activation_quantize.argtypes = [P, P, U, U, P]
        L.mi355_a8_enqueue_down_rawdots.argtypes = [P, P, U, P]
        L.mi355_a8_enqueue_down_rawdots_merge.argtypes = [P, P, P, P]
        L.mi355_a8_validate_union.argtypes = [P, P, DeviceBytes]
        L.mi355_a8_enqueue_probe_union.argtypes = [P, P, DeviceBytes, P]
        L.mi355_a8_validate_down_union.argtypes = [P, P, U, DeviceBytes]
        L.mi355_a8_enqueue_down_activation_quantize_union.argtypes = [P, P, U, DeviceBytes, U, P]
        L.mi355_a8_enqueue_down_rawdots_union.argtypes = [P, P, U, DeviceBytes, P]
        L.mi355_gguf_open.argtypes, L.mi355_gguf_open.restype = [C.c_char_p], P
        L.mi355_gguf_close.argtypes, L.mi355_gguf_close.restype = [P], None
        for name in ("tensor_count", "metadata_count", "alignment", "data_offset"):
            f = getattr(L, "mi355_gguf_" + name)
            f.argtypes, f.restype = [P], C.c_uint64
        L.mi355_gguf_tensor_at.argtypes = [P, C.c_uint64, P]
        L.mi355_gguf_find_tensor.argtypes = [P, C.c_char_p, P]
        L.mi355_gguf_metadata.argtypes = [P, C.c_char_p, P, P, P, P, P]
        L.mi355_gguf_moe_layer.argtypes = [P, U, P]
        L.mi355_executor_create.argtypes = [U, U, U]
        L.mi355_executor_create.restype = C.c_void_p
        L.mi355_executor_run.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi355_executor_destroy.argtypes = [C.c_void_p]
        L.mi355_executor_destroy.restype = None
        L.mi355_numerical_identity.restype = C.c_char_p
        L.mi355_numerical_identity.argtypes = [C.c_uint32, C.c_int]
        L.mi355_moe_plan_words.restype = C.c_size_t
        L.mi355_moe_plan_words.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32]
        L.mi355_moe_prefill_f16_workspace_bytes.restype = C.c_size_t
        L.mi355_moe_prefill_f16_workspace_bytes.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32]
        _lib = L
    return _lib


EXPORTS = ["mi355_last_error", "mi355_version", "mi355_numerical_identity", "mi355_dequantize_rows",
           "mi355_quantize_weight_rows", "mi355_quantize_a8", "mi355_gemv_q8_0_a8", "mi355_dense_a8_quantize", "mi355_gemv_q8_0_a8_chain", "mi355_moe_route",
           "mi355_moe_plan_words", "mi355_moe_enqueue_prologue", "mi355_moe_enqueue_csr", "mi355_moe_enqueue_project",
           "mi355_moe_enqueue_down", "mi355_moe_enqueue_merge", "mi355_moe_enqueue_combine", "mi355_moe_enqueue", "mi355_moe_enqueue_layer", "mi355_moe_enqueue_layer_front", "mi355_moe_enqueue_layer_back", "mi355_debug_early_route_perturb", "mi355_debug_down_merge_flat", "mi355_moe_enqueue_layer_normed", "mi355_moe_enqueue_layer_static", "mi355_static_workspace_prepare", "mi355_moe_enqueue_prefill_f16", "mi355_moe_enqueue_prefill_rows_f16", "mi355_moe_prefill_f16_workspace_bytes",
           "mi355_swiglu_quantize", "mi355_rmsnorm_f32", "mi355_shared_gate", "mi355_a8_validate", "mi355_a8_validate_down", "mi355_a8_enqueue_probe", "mi355_a8_enqueue_serial_prologue_probe", "mi355_a8_enqueue_quantize_only",
           "mi355_a8_enqueue_down_activation_quantize", "mi355_a8_enqueue_down_rawdots", "mi355_a8_enqueue_down_rawdots_merge",
           "mi355_a8_validate_union", "mi355_a8_enqueue_probe_union", "mi355_a8_validate_down_union",
           "mi355_a8_enqueue_down_activation_quantize_union", "mi355_a8_enqueue_down_rawdots_union",
           "mi355_moe_strided_enqueue_prologue", "mi355_moe_strided_enqueue_csr", "mi355_moe_strided_enqueue_project", "mi355_moe_strided_enqueue_down",
           "mi355_moe_strided_enqueue_merge", "mi355_moe_strided_enqueue_commit", "mi355_moe_strided_enqueue", "mi355_executor_create",
           "mi355_executor_run", "mi355_executor_destroy", "mi355_gguf_open", "mi355_gguf_close", "mi355_gguf_tensor_count",
           "mi355_gguf_metadata_count", "mi355_gguf_alignment", "mi355_gguf_data_offset", "mi355_gguf_tensor_at", "mi355_gguf_find_tensor",
           "mi355_gguf_metadata", "mi355_gguf_moe_layer"]


def require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU visible: the MI355X kernels cannot run (and nothing falls back to the CPU)")
    lib()


def check(rc):
    if rc != 0:
        raise StrixError(rc, lib().mi355_last_error().decode())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return C.c_void_p(0 if t is None else t.data_ptr())


def input_kind(t):
    return {torch.float32: INPUT_F32, torch.float16: INPUT_F16, torch.bfloat16: INPUT_BF16}[t.dtype]


def row_bytes(qtype, elements):
    return elements // 32 * Q8_0_BLOCK if qtype == TYPE_Q8_0 else elements // 256 * Q4_K_BLOCK


# ---------------------------------------------------------------------------------------------- thin wrappers
def dequantize_rows(qtype, packed, elements):
    packed = packed.contiguous().view(torch.uint8).reshape(-1, row_bytes(qtype, elements))
    out = torch.empty((packed.shape[0], elements), dtype=torch.float32, device=packed.device)
    check(lib().mi355_dequantize_rows(qtype, _p(packed), C.c_uint64(packed.shape[1]), packed.shape[0], elements, _p(out),
                                      C.c_uint64(elements), _stream()))
    return out


def quantize_weight_rows(qtype, x):
    x = x.contiguous()
    rows = x.numel() // x.shape[-1]
    out = torch.empty(x.shape[:-1] + (row_bytes(qtype, x.shape[-1]),), dtype=torch.uint8, device=x.device)
    check(lib().mi355_quantize_weight_rows(qtype, _p(x), rows, x.shape[-1], _p(out), _stream()))
    return out


def quantize_a8(x, want_sums=True):
    assert x.dim() == 2 and x.stride(1) == 1
    rows, width = x.shape
    codes = torch.empty((rows, width), dtype=torch.int8, device=x.device)
    deltas = torch.empty((rows, width // 32), dtype=torch.float32, device=x.device)
    sums = torch.empty((rows, width // 32), dtype=torch.int32, device=x.device) if want_sums else None
    status = torch.zeros(rows, dtype=torch.int32, device=x.device)
    check(lib().mi355_quantize_a8(_p(x), input_kind(x), rows, width, C.c_uint64(x.stride(0) * x.element_size()), _p(codes),
                                  _p(deltas), _p(sums), _p(status), _stream()))
    return codes, deltas, sums, status


def rmsnorm_f32(x, weight=None, eps=1e-6):
    """RMSNorm of fp32 rows in the reference's reduction order (strix::cpu::Kernels::rmsnorm_f32)."""
    assert x.dim() == 2 and x.is_contiguous() and x.dtype == torch.float32
    y = torch.empty_like(x)
    check(lib().mi355_rmsnorm_f32(_p(x), _p(weight), x.shape[1], C.c_float(eps), _p(y), x.shape[0], _stream()))
    return y


def shared_gate(x, scalar_weight, exp_kind=EXP_GFX1151, out=None):
    """gate[row] = sigmoid(dot(x[row], scalar_weight)) as the reference's shared-expert launcher computes it (mi355_shared_gate)."""
    rows, hidden = x.shape
    if out is None:
        out = torch.zeros((rows, 1), dtype=torch.float32, device=x.device)
    check(lib().mi355_shared_gate(_p(x), input_kind(x), rows, hidden, C.c_uint64(x.stride(0) * x.element_size()), _p(scalar_weight), exp_kind,
                                  _p(out), C.c_uint64(out.stride(0)), _stream()))
    return out


def gemv_q8_0_a8(weight, codes, deltas, n_in, count, out=None, accumulate=False, row_bytes_=None, out_stride=None):
    rows = codes.shape[0]
    if out is None:
        out = torch.zeros((rows, count), dtype=torch.float32, device=codes.device)
    v = Q8a8View(weight.data_ptr(), codes.data_ptr(), deltas.data_ptr(), out.data_ptr(),
                 row_bytes_ or n_in // 32 * Q8_0_BLOCK, n_in, count, rows, codes.shape[1], out_stride or out.shape[1], int(accumulate))
    check(lib().mi355_gemv_q8_0_a8(C.byref(v), _stream()))
    return out


def dense_a8_quantize(x):
    """The dense A8 profile's quantiser (mi355_dense_a8_quantize): a non-finite group gets delta = NaN and codes 0."""
    rows, width = x.shape
    codes = torch.zeros((rows, width), dtype=torch.int8, device=x.device)
    deltas = torch.zeros((rows, width // 32), dtype=torch.float32, device=x.device)
    check(lib().mi355_dense_a8_quantize(_p(x), input_kind(x), rows, width, C.c_uint64(x.stride(0) * x.element_size()), _p(codes), _p(deltas), _stream()))
    return codes, deltas


def gemv_q8_0_a8_chain(weight, codes, deltas, n_in, count):
    """Q8_0 x A8 with the dense A8 profile's row contract: one ascending fma chain per output (mi355_gemv_q8_0_a8_chain)."""
    rows = codes.shape[0]
    out = torch.zeros((rows, count), dtype=torch.float32, device=codes.device)
    v = Q8a8View(weight.data_ptr(), codes.data_ptr(), deltas.data_ptr(), out.data_ptr(), n_in // 32 * Q8_0_BLOCK, n_in, count, rows, codes.shape[1],
                 out.shape[1], 0)
    check(lib().mi355_gemv_q8_0_a8_chain(C.byref(v), _stream()))
    return out


def route(x, router_weight, top_k, bias=None, logits_order=LOGITS_FMA, renorm_eps=0.0, scale=1.0, renormalize=True, renorm_single=True,
          exp_kind=EXP_DECLARED, shared_experts=0, shared_slot_weights=None):
    rows, hidden = x.shape
    experts = router_weight.shape[0]
    p = RoutePolicy(experts, top_k, logits_order, renorm_eps, scale, int(renormalize), int(renorm_single), exp_kind, shared_experts,
                    None if shared_slot_weights is None else shared_slot_weights.data_ptr())
    ids = torch.empty((rows, top_k + shared_experts), dtype=torch.int32, device=x.device)
    weights = torch.empty((rows, top_k + shared_experts), dtype=torch.float32, device=x.device)
    scores = torch.empty((rows, experts), dtype=torch.float32, device=x.device)
    check(lib().mi355_moe_route(C.byref(p), _p(x), input_kind(x), rows, hidden, C.c_uint64(x.stride(0) * x.element_size()),
                                _p(router_weight), _p(bias), _p(ids), _p(weights), _p(scores), _stream()))
    return ids, weights, scores


def swiglu_quantize(gate, up, exp_kind=EXP_GFX1151, swiglu_limit=float("inf")):
    rows, ffn = gate.shape
    codes = torch.zeros((rows, ffn), dtype=torch.int8, device=gate.device)
    deltas = torch.zeros((rows, ffn // 32), dtype=torch.float32, device=gate.device)
    sums = torch.zeros((rows, ffn // 32), dtype=torch.int32, device=gate.device)
    h = torch.zeros((rows, ffn), dtype=torch.float32, device=gate.device)
    status = torch.zeros(rows, dtype=torch.int32, device=gate.device)
    check(lib().mi355_swiglu_quantize(_p(gate), _p(up), rows, ffn, exp_kind, C.c_float(swiglu_limit), _p(codes), _p(deltas), _p(sums), _p(h), _p(status), _stream()))
    return codes, deltas, sums, h, status


def combine(form, eo, w=None, base=None, round_eo=False):
    """The combine operator on its own (strix::moe_core::enqueue_combine, src/moe_core/route_wave_kernel.hpp:138-160):
    eo [rows][top_k][width] fp32, w [rows][top_k] or None (bf16-steps: unit weights), base [rows][width] or None."""
    rows, top_k, width = eo.shape
    y = torch.zeros((rows, width), dtype=torch.float32, device=eo.device)
    check(lib().mi355_moe_enqueue_combine(form, rows, top_k, width, _p(w), _p(eo), _p(base), _p(y), 1 if round_eo else 0, _stream()))
    return y


class A8Decode:
    """The reference's single-row A8 pipeline over the request / bindings entry points (include/strix/hip_moe_q4k_a8_probe.hpp:12,
    include/strix/hip_moe_a8_down.hpp:18-30): probe -> down_activation_quantize -> down_rawdots (+ slot merge). Owns the views the
    reference's caller owns (every one an allocation of its own, so the bundle is disjoint and 256-byte aligned) for up to
    `rows` logical rows. gate / up / down: uint8 device tensors holding every expert in GGUF order."""

    def __init__(self, hidden, intermediate, experts, top_k, gate, up, down, rows=1, gate_type=TYPE_Q4_K, down_type=TYPE_Q4_K, input_dtype=torch.bfloat16,
                 swiglu_limit=float("inf")):
        self.H, self.I, self.E, self.K, self.R = hidden, intermediate, experts, top_k, rows
        self.gate_type, self.down_type, self.limit = gate_type, down_type, swiglu_limit
        self.gate, self.up, self.down = gate, up, down
        d = gate.device
        z = lambda shape, dt: torch.zeros(shape, dtype=dt, device=d)
        self.input = z((rows, hidden), input_dtype)
        self.routes = z((rows, top_k), torch.int32)
        self.codes, self.deltas, self.sums = z((rows, hidden), torch.int8), z((rows, hidden // 32), torch.float32), z((rows, hidden // 32), torch.int32)
        self.status, self.aggregate = z(1, torch.int32), z(1, torch.int32)
        self.intermediates = z((rows, top_k, 2, intermediate), torch.float32)      # the probe's output = the down producer's input
        self.h_codes = z((rows, top_k, intermediate), torch.int8)
        self.h_deltas, self.h_sums = z((rows, top_k, intermediate // 32), torch.float32), z((rows, top_k, intermediate // 32), torch.int32)
        self.rawdots = z((rows, top_k, hidden), torch.float32)
        self.probe_identity = lib().mi355_numerical_identity(gate_type, 0)
        self.down_identity = lib().mi355_numerical_identity(down_type, 1)

    def request(self, rows=None):
        return A8Request(1, self.probe_identity, input_kind(self.input), A8Shape(self.H, self.I, self.E, self.K, rows or self.R), self.gate_type,
                         self.gate_type, 0, float("inf"))

    def bindings(self, rows=None):
        n = rows or self.R
        return A8Bindings(device_bytes(self.input[:n]), device_bytes(self.gate), device_bytes(self.up), device_bytes(self.routes[:n]),
                          device_bytes(self.codes[:n]), device_bytes(self.deltas[:n]), device_bytes(self.sums[:n]), device_bytes(self.status),
                          device_bytes(self.intermediates[:n]))

    def down_request(self):
        return A8DownRequest(1, self.down_identity, A8DownShape(self.H, self.I, self.E, self.K), self.down_type, self.limit)

    def down_bindings(self, rows=None, aggregate=True):
        n = rows or self.R
        return A8DownBindings(device_bytes(self.intermediates[:n]), device_bytes(self.down), device_bytes(self.routes[:n]), device_bytes(self.h_codes[:n]),
                              device_bytes(self.h_deltas[:n]), device_bytes(self.h_sums[:n]), device_bytes(self.rawdots[:n]), device_bytes(self.status),
                              device_bytes(self.aggregate if aggregate else None))

    def enqueue_probe(self, rows=None):
        q, b = self.request(rows), self.bindings(rows)
        check(lib().mi355_a8_enqueue_probe(C.byref(q), C.byref(b), _stream()))

    def enqueue_serial_prologue_probe(self, clear, clear_words, route_weights):
        req, b = self.request(1), self.bindings(1)
        check(lib().mi355_a8_enqueue_serial_prologue_probe(C.byref(req), C.byref(b), _p(clear), clear_words, _p(route_weights), _stream()))

    def enqueue_quantize_only(self):
        req, b = self.request(1), self.bindings(1)
        check(lib().mi355_a8_enqueue_quantize_only(C.byref(req), C.byref(b), _stream()))

    def enqueue_down_activation_quantize(self, rows=None, exp_kind=EXP_GFX1151):
        q, b = self.down_request(), self.down_bindings(rows)
        check(lib().mi355_a8_enqueue_down_activation_quantize(C.byref(q), C.byref(b), rows or self.R, exp_kind, _stream()))

    def enqueue_down_rawdots(self, rows=None):
        q, b = self.down_request(), self.down_bindings(rows)
        check(lib().mi355_a8_enqueue_down_rawdots(C.byref(q), C.byref(b), rows or self.R, _stream()))

    # ---- union rows form (include/strix/moe/expert_union.hpp): R <= 8 rows, every distinct expert read once
    def union_plan(self):
        """The caller's plan view: UNION_PLAN_BYTES of device memory, written by enqueue_probe_union."""
        if getattr(self, "plan", None) is None:
            self.plan = torch.zeros(UNION_PLAN_BYTES, dtype=torch.uint8, device=self.gate.device)
        return self.plan

    def enqueue_probe_union(self, rows=None):
        q, b = self.request(rows), self.bindings(rows)
        check(lib().mi355_a8_enqueue_probe_union(C.byref(q), C.byref(b), device_bytes(self.union_plan()), _stream()))

    def enqueue_down_activation_quantize_union(self, rows=None, exp_kind=EXP_GFX1151):
        q, b = self.down_request(), self.down_bindings(rows)
        check(lib().mi355_a8_enqueue_down_activation_quantize_union(C.byref(q), C.byref(b), rows or self.R, device_bytes(self.union_plan()), exp_kind, _stream()))

    def enqueue_down_rawdots_union(self, rows=None):
        q, b = self.down_request(), self.down_bindings(rows)
        check(lib().mi355_a8_enqueue_down_rawdots_union(C.byref(q), C.byref(b), rows or self.R, device_bytes(self.union_plan()), _stream()))

    def enqueue_down_rawdots_merge(self, route_weights, accumulation, output, record, domain=1, bf16_commit=False):
        """One row: rawdots, then the ordered slot merge, commit test and first-error record (SlotMergeTail)."""
        q, b = self.down_request(), self.down_bindings(1)
        tail = SlotMergeTail(None, _p(route_weights), _p(accumulation), _p(output), int(output.dtype == torch.bfloat16), int(bf16_commit), _p(record), domain)
        check(lib().mi355_a8_enqueue_down_rawdots_merge(C.byref(q), C.byref(b), C.byref(tail), _stream()))


class Executor:
    """The host executor's object on the GPU (strix::cpu::expert::Executor, src/cpu/core/routed_expert.hpp:79-95): create once,
    run(job) per step, destroy. Workspace for max_assignments x max_ffn is allocated at construction; run allocates nothing."""

    def __init__(self, max_assignments, max_ffn, exp_kind=EXP_GFX1151):
        self.handle = lib().mi355_executor_create(max_assignments, max_ffn, exp_kind)
        if not self.handle:
            raise StrixError(E_INVALID_ARGUMENT, lib().mi355_last_error().decode())

    def run(self, job):
        check(lib().mi355_executor_run(self.handle, C.byref(job), _stream()))

    def close(self):
        if self.handle:
            lib().mi355_executor_destroy(self.handle)
            self.handle = None

    def __del__(self):
        self.close()


class MoeLayer:
    """One MoE layer's expert tensors plus caller-owned work buffers for up to max_rows rows (the reference's
    Rows / Weights bundle, include/strix/cuda/qwen_moe.hpp:55-93)."""

    def __init__(self, hidden, ffn, experts, top_k, gate, up, down, max_rows, exp_kind=EXP_GFX1151, intermediates=False,
                 gate_expert_stride=0, gate_row_stride=0, down_expert_stride=0, down_row_stride=0, prefill_f16=False,
                 gate_type=TYPE_Q4_K, down_type=TYPE_Q4_K, output_stride=None, swiglu_limit=float("inf")):
        dev = gate.device
        self.hidden, self.ffn, self.experts, self.top_k, self.max_rows = hidden, ffn, experts, top_k, max_rows
        self.gate, self.up, self.down = gate, up, down
        self.w = MoeWeights(hidden, ffn, experts, top_k, gate_type, down_type, gate.data_ptr(), up.data_ptr(), down.data_ptr(),
                            gate_expert_stride, gate_row_stride, down_expert_stride, down_row_stride, exp_kind, swiglu_limit)
        n = max_rows * top_k
        z = lambda shape, dt: torch.zeros(shape, dtype=dt, device=dev)
        self.codes, self.deltas, self.sums = z((max_rows, hidden), torch.int8), z((max_rows, hidden // 32), torch.float32), z((max_rows, hidden // 32), torch.int32)
        self.status, self.job_status = z(max_rows, torch.int32), z(4, torch.int32)
        self.down_codes, self.down_deltas, self.down_sums = z((n, ffn), torch.int8), z((n, ffn // 32), torch.float32), z((n, ffn // 32), torch.int32)
        self.rawdots = z((max_rows, top_k, hidden), torch.float32)
        self.output_stride = output_stride or hidden          # floats between output rows (>= hidden)
        self.output = z((max_rows, self.output_stride), torch.float32)[:, :hidden]
        self.gate_out = z((n, ffn), torch.float32) if intermediates else None
        self.up_out = z((n, ffn), torch.float32) if intermediates else None
        self.h_out = z((n, ffn), torch.float32) if intermediates else None
        self.plan = z(int(lib().mi355_moe_plan_words(experts, max_rows, top_k)), torch.int32)
        # workspace of the fp16 MFMA prefill form: h in fp16 and the sub-block sums of h and of the input rows
        self.h_f16 = z((int(lib().mi355_moe_prefill_f16_workspace_bytes(hidden, ffn, max_rows, top_k)),), torch.uint8) if prefill_f16 else None

    def rows_view(self, x, ids, weights, base=None):
        rows = x.shape[0]
        assert rows <= self.max_rows and x.stride(1) == 1
        self._keep = (x, ids, weights, base)
        return rows, MoeRows(x.data_ptr(), input_kind(x), x.stride(0) * x.element_size(), ids.data_ptr(), weights.data_ptr(),
                             self.codes.data_ptr(), self.deltas.data_ptr(), self.sums.data_ptr(), self.status.data_ptr(),
                             _p(self.gate_out).value or 0, _p(self.up_out).value or 0, _p(self.h_out).value or 0,
                             self.down_codes.data_ptr(), self.down_deltas.data_ptr(), self.down_sums.data_ptr(),
                             self.rawdots.data_ptr(), 0 if base is None else base.data_ptr(), self.output.data_ptr(), self.output_stride,
                             self.plan.data_ptr(), self.job_status.data_ptr(), _p(self.h_f16).value or 0)

    def run(self, x, ids, weights, base=None, combine=COMBINE_FMA_SLOT):
        rows, rv = self.rows_view(x, ids, weights, base)
        check(lib().mi355_moe_enqueue(C.byref(self.w), C.byref(rv), rows, combine, _stream()))
        return self.output[:rows]

    def run_prefill_f16(self, x, ids, weights, base=None, combine=COMBINE_FMA_SLOT):
        """The routed experts on the matrix cores (fp16 weights x fp16 rows, fp32 accumulation): mi355_moe_enqueue_prefill_f16."""
        rows, rv = self.rows_view(x, ids, weights, base)
        check(lib().mi355_moe_enqueue_prefill_f16(C.byref(self.w), C.byref(rv), rows, combine, _stream()))
        if combine == COMBINE_NONE:      # no combine: the unweighted per-slot outputs [rows][top_k][hidden]
            return self.rawdots[:rows]
        return self.output[:rows]

    def run_prefill_rows_f16(self, views, rows, clear_words=0):
        """mi355_moe_enqueue_prefill_rows_f16 over caller-built strided views (PrefillRows); plan / job word / h_f16 default to this
        layer's own buffers."""
        if not views.plan:
            views.plan, views.job_status, views.h_f16 = self.plan.data_ptr(), self.job_status.data_ptr(), self.h_f16.data_ptr()
        check(lib().mi355_moe_enqueue_prefill_rows_f16(C.byref(self.w), C.byref(views), rows, clear_words, _stream()))

    def run_layer(self, x, router_weight, bias=None, base=None, combine=COMBINE_FMA_SLOT, logits_order=LOGITS_FMA, renorm_eps=0.0,
                  scale=1.0, renormalize=True, renorm_single=True, exp_kind=EXP_DECLARED, shared_experts=0, norm=None, half=None, shared_slot_weights=None):
        """Router + experts + combine through mi355_moe_enqueue_layer. Returns (output, ids, weights, scores).
        shared_experts: the last `shared_experts` experts of the tensors are always on (the router picks among the others);
        shared_slot_weights [rows][shared_experts]: their weights in the place of 1 (the sigmoid gate of shared_gate()).
        norm: (weight or None, eps) - the RMSNorm of x runs inside the first launch (mi355_moe_enqueue_layer_normed); the
        normalised rows are left in self.normed."""
        rows = x.shape[0]
        if router_weight.shape[0] != self.experts - shared_experts or router_weight.shape[1] != self.hidden:
            raise StrixError(E_INVALID_ARGUMENT, "the router weight must be [experts - shared_experts][hidden]")
        if not hasattr(self, "ids") or self.ids.shape[0] < rows:
            self.ids = torch.zeros((self.max_rows, self.top_k), dtype=torch.int32, device=x.device)
            self.route_w = torch.zeros((self.max_rows, self.top_k), dtype=torch.float32, device=x.device)
            self.scores = torch.zeros((self.max_rows, self.experts), dtype=torch.float32, device=x.device)
        _, rv = self.rows_view(x, self.ids, self.route_w, base)
        p = RoutePolicy(self.experts - shared_experts, self.top_k - shared_experts, logits_order, renorm_eps, scale, int(renormalize), int(renorm_single),
                        exp_kind, shared_experts, None if shared_slot_weights is None else shared_slot_weights.data_ptr())
        if norm is None:
            # half: "front" / "back" = the layer's two halves as calls of their own (mi355_moe_enqueue_layer_front / _back)
            entry = lib().mi355_moe_enqueue_layer if half is None else getattr(lib(), "mi355_moe_enqueue_layer_" + half)
            check(entry(C.byref(p), _p(router_weight), _p(bias), _p(self.scores), C.byref(self.w), C.byref(rv), rows, combine, _stream()))
        else:
            if not hasattr(self, "normed"):
                self.normed = torch.zeros((self.max_rows, self.hidden), dtype=torch.float32, device=x.device)
            check(lib().mi355_moe_enqueue_layer_normed(C.byref(p), _p(router_weight), _p(bias), _p(self.scores), _p(norm[0]), C.c_float(norm[1]),
                                                       _p(self.normed), C.byref(self.w), C.byref(rv), rows, combine, _stream()))
        return self.output[:rows], self.ids[:rows], self.route_w[:rows], self.scores[:rows]

    def run_layer_static(self, x, router_weight, ids, route_w, status, output, bias=None, base=None, combine=COMBINE_FMA_SLOT):
        """mi355_moe_enqueue_layer_static: the work buffers are the library's own; only inputs and outputs are passed."""
        rows = x.shape[0]
        p = RoutePolicy(self.experts, self.top_k, LOGITS_FMA, 0.0, 1.0, 1, 1, EXP_DECLARED)
        check(lib().mi355_moe_enqueue_layer_static(C.byref(p), _p(router_weight), _p(bias), C.byref(self.w), _p(x), input_kind(x),
                                                   C.c_uint64(x.stride(0) * x.element_size()), rows, _p(ids), _p(route_w), _p(status), _p(base),
                                                   _p(output), C.c_uint64(output.stride(0)), combine, _stream()))
        return output[:rows]

    def stage(self, name, x, ids, weights, base=None, combine=COMBINE_FMA_SLOT):
        rows, rv = self.rows_view(x, ids, weights, base)
        fn = getattr(lib(), "mi355_moe_enqueue_" + name)
        if name == "merge":
            check(fn(C.byref(self.w), C.byref(rv), rows, combine, _stream()))
        else:
            check(fn(C.byref(self.w), C.byref(rv), rows, _stream()))
