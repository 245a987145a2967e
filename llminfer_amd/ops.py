"""Torch-tensor front end of the C ABI. PyTorch is only used for device memory
and streams: each function reads data_ptr()s and calls libllmi_hip.so."""
import ctypes

import torch

from . import _binding as B

_BF16_DTYPES = (torch.bfloat16, torch.uint16, torch.int16)


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream_handle(stream):
    if stream is None:
        stream = torch.cuda.current_stream()
    return stream.cuda_stream if hasattr(stream, "cuda_stream") else int(stream)


def _check_dev(name, t, dtypes):
    if t is None:
        return
    if not t.is_cuda:
        raise ValueError("%s must be a device tensor" % name)
    if t.dtype not in dtypes:
        raise ValueError("%s has dtype %s, expected one of %s" % (name, t.dtype, dtypes))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)


def workspace_bytes(head_num, head_dim, max_seq_len):
    return int(B.lib().llmi_hip_mha_workspace_bytes(head_num, head_dim, max_seq_len))


def make_mha_args(query, key_cache, value_cache, output, workspace, *, layer_id, pos, kv_dim, kv_mul,
                  head_num, head_dim, max_seq_len, kv_layout=B.KV_LAYOUT_POS_MAJOR, force_path=B.PATH_AUTO,
                  num_splits=0, waves_per_group=0, output_f32=None, stream=None, pos_device=None, workspace_side=0):
    """Fills an llmi_mha_args from torch tensors (or raw integer addresses)."""
    def addr(x):
        return x if (x is None or isinstance(x, int)) else x.data_ptr()

    a = B.MhaArgs()
    a.query = addr(query)
    a.key_cache = addr(key_cache)
    a.value_cache = addr(value_cache)
    a.workspace = addr(workspace)
    if workspace is None:
        a.workspace_bytes = 0
    elif isinstance(workspace, int):
        raise ValueError("pass workspace as a tensor so its size is known")
    else:
        a.workspace_bytes = workspace.numel() * workspace.element_size()
    a.output = addr(output)
    a.output_f32 = addr(output_f32)
    a.layer_id, a.pos, a.kv_dim, a.kv_mul = layer_id, pos, kv_dim, kv_mul
    a.head_num, a.head_dim, a.max_seq_len = head_num, head_dim, max_seq_len
    a.kv_layout, a.force_path, a.num_splits, a.waves_per_group = kv_layout, force_path, num_splits, waves_per_group
    a.stream = stream
    a.pos_device = addr(pos_device)
    a.workspace_side = workspace_side
    return a


def workspace_side(workspace, stream=None):
    """Which 8 KiB blocks of `workspace` lie near which side of the package (llmi_hip_mha_workspace_side): 0, 1 or 2,
    to be passed as workspace_side with this workspace. Overwrites its first 32 KiB and synchronises the stream."""
    _check_dev("workspace", workspace, (torch.float32,))
    side = ctypes.c_int32(0)
    s = stream if stream is not None else torch.cuda.current_stream(workspace.device).cuda_stream
    B.check(B.lib().llmi_hip_mha_workspace_side(workspace.data_ptr(), workspace.numel() * workspace.element_size(), s,
                                                ctypes.byref(side)), "llmi_hip_mha_workspace_side")
    return side.value


def mha_plan(args):
    plan = B.MhaPlan()
    B.check(B.lib().llmi_hip_mha_plan(ctypes.byref(args), ctypes.byref(plan)), "llmi_hip_mha_plan")
    return plan


def mha_decode(query, key_cache, value_cache, output, workspace, *, stream=None, **kw):
    """Decode attention for one layer / one token on the current (or given) stream."""
    _check_dev("query", query, _BF16_DTYPES)
    _check_dev("key_cache", key_cache, _BF16_DTYPES)
    _check_dev("value_cache", value_cache, _BF16_DTYPES)
    _check_dev("output", output, _BF16_DTYPES)
    _check_dev("workspace", workspace, (torch.float32,))
    _check_dev("output_f32", kw.get("output_f32"), (torch.float32,))
    args = make_mha_args(query, key_cache, value_cache, output, workspace,
                         stream=_stream_handle(stream), **kw)
    B.check(B.lib().llmi_hip_mha_decode(ctypes.byref(args)), "llmi_hip_mha_decode")
    return output


def mha_decode_raw(args):
    """Calls llmi_hip_mha_decode on a prepared llmi_mha_args; returns the status."""
    return int(B.lib().llmi_hip_mha_decode(ctypes.byref(args)))


def qk_norm_rope_append(query, key_new, value_new, key_cache, value_cache, norm_weight, sin_cache, cos_cache, *,
                        layer_id, pos, kv_dim, head_num, head_dim, max_seq_len,
                        kv_layout=B.KV_LAYOUT_POS_MAJOR, eps=1e-6, query_src=None, stream=None):
    for name, t in (("query", query), ("query_src", query_src), ("key_new", key_new), ("value_new", value_new),
                    ("key_cache", key_cache), ("value_cache", value_cache), ("norm_weight", norm_weight)):
        _check_dev(name, t, _BF16_DTYPES)
    _check_dev("sin_cache", sin_cache, (torch.float32,))
    _check_dev("cos_cache", cos_cache, (torch.float32,))
    a = B.QkNormRopeArgs()
    a.query, a.query_src, a.key_new, a.value_new = _ptr(query), _ptr(query_src), _ptr(key_new), _ptr(value_new)
    a.key_cache, a.value_cache, a.norm_weight = _ptr(key_cache), _ptr(value_cache), _ptr(norm_weight)
    a.sin_cache, a.cos_cache = _ptr(sin_cache), _ptr(cos_cache)
    a.layer_id, a.pos, a.kv_dim, a.head_num = layer_id, pos, kv_dim, head_num
    a.head_dim, a.max_seq_len, a.kv_layout, a.eps = head_dim, max_seq_len, kv_layout, eps
    a.stream = _stream_handle(stream)
    B.check(B.lib().llmi_hip_qk_norm_rope_append(ctypes.byref(a)), "llmi_hip_qk_norm_rope_append")


def mha_decode_append(query_raw, key_new, value_new, norm_weight, sin_cache, cos_cache, key_cache, value_cache,
                      output, workspace, *, eps=1e-6, stream=None, o_weight=None, residual=None, one_launch=False, **kw):
    """QK-Norm + RoPE + K/V append + decode attention as one kernel (llmi_hip_mha_decode_append). With `o_weight`
    [hidden][head_num*128] and `residual` [hidden]: llmi_hip_mha_decode_append_oproj (`one_launch`: ask for its
    one-launch form); returns the launch count."""
    for name, t in (("query_raw", query_raw), ("key_new", key_new), ("value_new", value_new),
                    ("norm_weight", norm_weight), ("key_cache", key_cache), ("value_cache", value_cache),
                    ("output", output)):
        _check_dev(name, t, _BF16_DTYPES)
    for name, t in (("sin_cache", sin_cache), ("cos_cache", cos_cache), ("workspace", workspace),
                    ("output_f32", kw.get("output_f32"))):
        _check_dev(name, t, (torch.float32,))
    a = B.MhaAppendArgs()
    a.mha = make_mha_args(query_raw, key_cache, value_cache, output, workspace, stream=_stream_handle(stream), **kw)
    a.key_new, a.value_new, a.norm_weight = _ptr(key_new), _ptr(value_new), _ptr(norm_weight)
    a.sin_cache, a.cos_cache, a.eps = _ptr(sin_cache), _ptr(cos_cache), eps
    if o_weight is None:
        B.check(B.lib().llmi_hip_mha_decode_append(ctypes.byref(a)), "llmi_hip_mha_decode_append")
        return output
    # ... with the layer's output projection and residual add behind it (llmi_hip_mha_decode_append_oproj)
    _check_dev("o_weight", o_weight, _BF16_DTYPES)
    _check_dev("residual", residual, _BF16_DTYPES)
    t = B.AttnOprojArgs()
    t.attn, t.o_weight, t.residual, t.hidden = a, _ptr(o_weight), _ptr(residual), residual.numel()
    t.one_launch = 1 if one_launch else 0
    launches = B.lib().llmi_hip_mha_oproj_launches(ctypes.byref(t))
    B.check(B.lib().llmi_hip_mha_decode_append_oproj(ctypes.byref(t)), "llmi_hip_mha_decode_append_oproj")
    return launches


def mha_decode_append_stack(query_raw, key_new, value_new, norm_weight, sin_cache, cos_cache, key_cache, value_cache,
                            output, workspace, *, layer_count, query_stride, key_new_stride, value_new_stride,
                            norm_weight_stride, output_stride, eps=1e-6, stream=None, **kw):
    """llmi_hip_mha_decode_append for `layer_count` consecutive layers (llmi_hip_mha_decode_append_stack): the tensors
    are the first layer's, layer l uses them moved on by l strides (elements). Returns the launch count."""
    for name, t in (("query_raw", query_raw), ("key_new", key_new), ("value_new", value_new),
                    ("norm_weight", norm_weight), ("key_cache", key_cache), ("value_cache", value_cache),
                    ("output", output)):
        _check_dev(name, t, _BF16_DTYPES)
    for name, t in (("sin_cache", sin_cache), ("cos_cache", cos_cache), ("workspace", workspace),
                    ("output_f32", kw.get("output_f32"))):
        _check_dev(name, t, (torch.float32,))
    t = B.MhaStackArgs()
    a = t.first
    a.mha = make_mha_args(query_raw, key_cache, value_cache, output, workspace, stream=_stream_handle(stream), **kw)
    a.key_new, a.value_new, a.norm_weight = _ptr(key_new), _ptr(value_new), _ptr(norm_weight)
    a.sin_cache, a.cos_cache, a.eps = _ptr(sin_cache), _ptr(cos_cache), eps
    t.layer_count = layer_count
    t.query_stride, t.key_new_stride, t.value_new_stride = query_stride, key_new_stride, value_new_stride
    t.norm_weight_stride, t.output_stride = norm_weight_stride, output_stride
    launches = B.lib().llmi_hip_mha_stack_launches(ctypes.byref(t))
    B.check(B.lib().llmi_hip_mha_decode_append_stack(ctypes.byref(t)), "llmi_hip_mha_decode_append_stack")
    return launches


def sincos_table(head_dim, max_seq_len, device="cuda", stream=None):
    sin = torch.empty((max_seq_len, head_dim // 2), dtype=torch.float32, device=device)
    cos = torch.empty_like(sin)
    B.check(B.lib().llmi_hip_sincos_table(sin.data_ptr(), cos.data_ptr(), head_dim, max_seq_len,
                                          _stream_handle(stream)), "llmi_hip_sincos_table")
    return sin, cos


def kv_restride(src_pos_major, dst_head_major, *, layer_num, max_seq_len, kv_dim, head_dim, num_pos, stream=None):
    _check_dev("src", src_pos_major, _BF16_DTYPES)
    _check_dev("dst", dst_head_major, _BF16_DTYPES)
    if dst_head_major.numel() < src_pos_major.numel():
        raise ValueError("destination cache is smaller than the source")
    B.check(B.lib().llmi_hip_kv_restride(src_pos_major.data_ptr(), dst_head_major.data_ptr(), layer_num,
                                         max_seq_len, kv_dim, head_dim, num_pos, _stream_handle(stream)),
            "llmi_hip_kv_restride")
    return dst_head_major


def gemv(input, weight, output, *, mode=B.GEMV_OUT_BF16, stream=None):
    """output = weight @ input (bf16 [n][k] x bf16 [k], fp32 accumulate): bf16 or fp32 output, or the
    bf16 residual in `output` updated in place (llmi_hip_gemv)."""
    _check_dev("input", input, _BF16_DTYPES)
    _check_dev("weight", weight, _BF16_DTYPES)
    _check_dev("output", output, (torch.float32,) if mode == B.GEMV_OUT_F32 else _BF16_DTYPES)
    a = B.GemvArgs()
    a.input, a.weight, a.output = _ptr(input), _ptr(weight), _ptr(output)
    a.n, a.k, a.mode = weight.shape[0], weight.shape[1], mode
    a.stream = _stream_handle(stream)
    B.check(B.lib().llmi_hip_gemv(ctypes.byref(a)), "llmi_hip_gemv")
    return output


def qkv_gemv(input, weight, query, key, value, *, stream=None):
    """The packed QKV projection: rows [0, dim) of weight @ input go to query, the next kv_dim to key,
    the last kv_dim to value (llmi_hip_qkv_gemv)."""
    for name, t in (("input", input), ("weight", weight), ("query", query), ("key", key), ("value", value)):
        _check_dev(name, t, _BF16_DTYPES)
    a = B.QkvGemvArgs()
    a.input, a.weight, a.query, a.key, a.value = _ptr(input), _ptr(weight), _ptr(query), _ptr(key), _ptr(value)
    a.dim, a.kv_dim, a.k = query.numel(), key.numel(), weight.shape[1]
    assert value.numel() == key.numel() and weight.shape[0] == a.dim + 2 * a.kv_dim
    a.stream = _stream_handle(stream)
    B.check(B.lib().llmi_hip_qkv_gemv(ctypes.byref(a)), "llmi_hip_qkv_gemv")
