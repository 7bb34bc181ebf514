"""The plain C++ references of the kernels (csrc/reference/reference.cpp), called through ctypes on float32
tensors in host memory, with the method names of the kernel library's Python face."""
import ctypes

import torch


def _p(tensor):
    return ctypes.c_void_p(0 if tensor is None else tensor.data_ptr())


def _f32(tensor):
    return None if tensor is None else tensor.detach().to("cpu", torch.float32).contiguous()


def _i32(tensor):
    return None if tensor is None else tensor.detach().to("cpu", torch.int32).contiguous()


class CppReference:
    name = "c++ reference"

    def __init__(self):
        from xeno_rt_amd.ops import build
        path = build.find_reference_library() or build.build_reference(verbose=False)
        self.lib = ctypes.CDLL(path)
        for name in ("xrt_ref_embed", "xrt_ref_add", "xrt_ref_rmsnorm", "xrt_ref_linear", "xrt_ref_qkv_prepare",
                     "xrt_ref_attention", "xrt_ref_sample", "xrt_ref_random_normal", "xrt_ref_pack_weight"):
            getattr(self.lib, name).restype = None

    def embed(self, table, ids):
        table, ids = _f32(table), _i32(ids)
        out = torch.empty(ids.shape[0], table.shape[1])
        self.lib.xrt_ref_embed(_p(table), _p(ids), _p(out), ids.shape[0], table.shape[1])
        return out

    def rmsnorm(self, x, weight, eps, rows=None):
        x, weight, rows = _f32(x), _f32(weight), _i32(rows)
        count = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty(count, x.shape[1])
        self.lib.xrt_ref_rmsnorm(_p(x), _p(weight), ctypes.c_float(eps), _p(out), _p(rows), count, x.shape[1])
        return out

    def linear(self, a, w, base=None):
        """a w^T, added to `base` if given."""
        a, w = _f32(a), _f32(w)
        out = torch.zeros(a.shape[0], w.shape[0]) if base is None else _f32(base).clone()
        self.lib.xrt_ref_linear(_p(a), _p(w), _p(out), a.shape[0], w.shape[0], a.shape[1], 0 if base is None else 1)
        return out

    def linear_glu(self, a, w_gate_up):
        a, w = _f32(a), _f32(w_gate_up)
        out = torch.empty(a.shape[0], w.shape[0] // 2)
        self.lib.xrt_ref_linear(_p(a), _p(w), _p(out), a.shape[0], w.shape[0] // 2, a.shape[1], 2)
        return out

    def qkv_prepare(self, qkv, n_heads, n_kv_heads, head_dim, positions, slots, q_norm=None, k_norm=None, norm_eps=0.0,
                    rope_theta=None, rope_dim=0, rope_scale=1.0, kv=None):
        """Returns the prepared rows; with kv = (k, v, block_table) as float32 host tensors, writes into them."""
        out = _f32(qkv).clone()
        positions, slots = _i32(positions), _i32(slots)
        q_norm, k_norm, rope_theta = _f32(q_norm), _f32(k_norm), _f32(rope_theta)
        k = v = table = None
        stride = blocks = 0
        if kv is not None:
            k, v, table = kv
            assert k.dtype == torch.float32 and v.dtype == torch.float32 and table.dtype == torch.int32
            stride, blocks = table.shape[1], k.shape[0]
        self.lib.xrt_ref_qkv_prepare(_p(out), out.shape[0], n_heads, n_kv_heads, head_dim, _p(positions), _p(slots),
                                     _p(q_norm), _p(k_norm), ctypes.c_float(norm_eps), _p(rope_theta), int(rope_dim),
                                     ctypes.c_float(rope_scale), _p(k), _p(v), _p(table), stride, blocks)
        return out

    def attention(self, qkv, n_heads, n_kv_heads, head_dim, k, v, block_table, positions, slots, scale, window=0, distance_slopes=None):
        qkv, k, v = _f32(qkv), _f32(k), _f32(v)
        table, positions, slots = _i32(block_table), _i32(positions), _i32(slots)
        out = torch.empty(qkv.shape[0], n_heads * head_dim)
        self.lib.xrt_ref_attention(_p(qkv), qkv.shape[0], n_heads, n_kv_heads, head_dim, _p(k), _p(v), _p(table),
                                   table.shape[1], _p(positions), _p(slots), _p(out), ctypes.c_float(scale), int(window or 0),
                                   _p(_f32(distance_slopes)) if distance_slopes is not None else None)
        return out

    def sample(self, logits, temperature, top_k, top_p, penalty, history, history_spans, uniforms):
        logits = _f32(logits)
        rows, vocab = logits.shape
        out = torch.empty(rows, dtype=torch.int32)
        args = [_f32(torch.as_tensor(temperature)), _i32(torch.as_tensor(top_k)), _f32(torch.as_tensor(top_p)),
                _f32(torch.as_tensor(penalty)), _i32(torch.as_tensor(history)), _i32(torch.as_tensor(history_spans))]
        uniforms = _f32(torch.as_tensor(uniforms))
        self.lib.xrt_ref_sample(_p(logits), rows, vocab, _p(out), *[_p(a) for a in args], None, _p(uniforms))
        return out.tolist()

    def random_normal(self, count, key, scale, offset=0.0):
        out = torch.empty(count)
        self.lib.xrt_ref_random_normal(_p(out), ctypes.c_long(count), ctypes.c_ulonglong(key), ctypes.c_float(scale),
                                       ctypes.c_float(offset))
        return out

    def pack(self, w, kind=1, gated_n=0, head_dim=0, rotated_heads=0):
        w = _f32(w)
        out = torch.empty((w.shape[0] + 15) // 16 * 16 * w.shape[1])
        self.lib.xrt_ref_pack_weight(_p(w), _p(out), w.shape[0], w.shape[1], kind, gated_n, head_dim, rotated_heads)
        return out
