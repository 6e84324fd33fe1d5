"""Torch-facing wrappers of the C ABI: device tensors in, device tensors out, nothing computed in Python.

PyTorch is used for device memory and the current stream only.  Every function raises if libtka.so is
missing or a call is rejected; there is no CPU or eager fallback.
"""
import ctypes as C

import torch

from . import _lib as L

_DT = {torch.float16: L.TKA_F16, torch.bfloat16: L.TKA_BF16}
_workspaces = {}


def _dtype_code(t):
    if t.dtype not in _DT:
        raise TypeError("expected float16 or bfloat16, got %s" % t.dtype)
    return _DT[t.dtype]


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _workspace(nbytes, device):
    """Workspace of the one-shot wrappers: one growing byte buffer per (device, stream), looked up by the stream the
    call is about to be launched on; calls on one stream are ordered, so they may share it.  Never grown during a
    graph capture (the allocation would belong to the capture's pool and be handed to later eager calls)."""
    key = (device.index, torch.cuda.current_stream().cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("the workspace of this stream must exist before a graph capture: call once eagerly, "
                               "or use a plan object (it owns its workspace)")
        buf = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def _own_workspace(nbytes, device):
    """Workspace of a plan object: its own buffer, so that plans run on different streams never share one."""
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def _need_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("tensors must live on the GPU")


def _kv_strides(kv, batch):
    """kv is [N, H, 128] (shared by the batch) or [B, N, H, 128]; returns (stride_b, stride_n, stride_h, N, H)."""
    if kv.stride(-1) != 1 or kv.shape[-1] != 128:
        raise ValueError("last dim must be 128 and contiguous")
    if kv.dim() == 3:
        return 0, kv.stride(0), kv.stride(1), kv.shape[0], kv.shape[1]
    if kv.dim() == 4:
        if kv.shape[0] != batch:
            raise ValueError("batch mismatch")
        return kv.stride(0), kv.stride(1), kv.stride(2), kv.shape[1], kv.shape[2]
    raise ValueError("keys/values must be [N,H,128] or [B,N,H,128]")


def _q3(q):
    if q.dim() == 2:
        q = q.unsqueeze(0)
    if q.dim() != 3 or q.shape[-1] != 128 or q.stride(-1) != 1 or q.stride(1) != 128:
        raise ValueError("q must be [B,Hq,128] with contiguous heads")
    return q


class GemvTopkPlan:
    """Argument block, outputs and workspace of one fused GEMV + top-k configuration; run() is one C call."""

    def __init__(self, q, keys, k, group=1, scale=1.0, num_chunks=1, return_scores=False, score_mode=L.TKA_SCORE_CANONICAL):
        _need_cuda(q, keys)
        q = _q3(q)
        B = q.shape[0]
        sb, sn, sh, N, H = _kv_strides(keys, B)
        if q.shape[1] != H * group:
            raise ValueError("q heads != kv heads * group")
        self.q, self.keys = q, keys
        self.idx = torch.empty((B, H, num_chunks * k), dtype=torch.int32, device=q.device)
        self.val = torch.empty((B, H, num_chunks * k), dtype=torch.float32, device=q.device)
        self.scores = torch.empty((B, H, N), dtype=torch.float32, device=q.device) if return_scores else None
        a = L.GemvTopkArgs()
        a.q, a.keys = q.data_ptr(), keys.data_ptr()
        a.dtype, a.batch, a.num_kv_heads, a.group, a.head_dim = _dtype_code(keys), B, H, group, 128
        a.k, a.num_chunks, a.seq_len, a.score_mode = k, num_chunks, N, score_mode
        a.q_stride_b, a.key_stride_b, a.key_stride_n, a.key_stride_h = q.stride(0), sb, sn, sh
        a.scale = scale
        a.out_idx, a.out_val = self.idx.data_ptr(), self.val.data_ptr()
        a.out_scores = self.scores.data_ptr() if self.scores is not None else None
        need = L.lib().tka_gemv_topk_workspace_bytes(C.byref(a))
        self.ws = _own_workspace(need, q.device)
        a.workspace, a.workspace_bytes = self.ws.data_ptr(), self.ws.numel()
        self.args = a
        self._fn = L.lib().tka_gemv_topk

    def run(self):
        self.args.stream = torch.cuda.current_stream().cuda_stream
        L.check(self._fn(C.byref(self.args)), "tka_gemv_topk")
        return self

    def redone_segments(self):
        """Diagnostic: segments of the last run() that the selection kernel had to redo from the keys."""
        n = C.c_int32(0)
        L.check(L.lib().tka_gemv_topk_redone_segments(C.byref(self.args), C.byref(n)), "tka_gemv_topk_redone_segments")
        return n.value

    def gave_up_slices(self):
        """Diagnostic: candidate slices of the last run() whose workgroup ran out of its wait for the threshold."""
        n = C.c_int32(0)
        L.check(L.lib().tka_gemv_topk_gave_up_slices(C.byref(self.args), C.byref(n)), "tka_gemv_topk_gave_up_slices")
        return n.value


def gemv_topk(q, keys, k, group=1, scale=1.0, num_chunks=1, return_scores=False, score_mode=L.TKA_SCORE_CANONICAL):
    """Fused GEMV + top-k.  Returns (idx int32 [B,Hkv,num_chunks*k], val fp32 same shape[, scores fp32 [B,Hkv,N]])."""
    plan = GemvTopkPlan(q, keys, k, group, scale, num_chunks, return_scores, score_mode).run()
    return (plan.idx, plan.val, plan.scores) if return_scores else (plan.idx, plan.val)


def gemv_scores(q, keys, group=1, scale=1.0, score_mode=L.TKA_SCORE_CANONICAL):
    """GEMV phase alone: fp32 scores [B,Hkv,N]."""
    _need_cuda(q, keys)
    q = _q3(q)
    B = q.shape[0]
    sb, sn, sh, N, H = _kv_strides(keys, B)
    scores = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
    a = L.GemvTopkArgs()
    a.q, a.keys = q.data_ptr(), keys.data_ptr()
    a.dtype, a.batch, a.num_kv_heads, a.group, a.head_dim = _dtype_code(keys), B, H, group, 128
    a.k, a.num_chunks, a.seq_len, a.score_mode = 1, 1, N, score_mode
    a.q_stride_b, a.key_stride_b, a.key_stride_n, a.key_stride_h = q.stride(0), sb, sn, sh
    a.scale = scale
    a.out_scores = scores.data_ptr()
    a.stream = _stream()
    L.check(L.lib().tka_gemv_scores(C.byref(a)), "tka_gemv_scores")
    return scores


def topk(scores, k):
    """Selection phase alone on fp32 scores [S, N] (row stride free).  Returns (idx int32 [S,k], val fp32 [S,k])."""
    _need_cuda(scores)
    if scores.dim() == 1:
        scores = scores.unsqueeze(0)
    if scores.dtype != torch.float32 or scores.dim() != 2 or scores.stride(1) != 1:
        raise ValueError("scores must be fp32 [S,N] with contiguous rows")
    S, N = scores.shape
    idx = torch.empty((S, k), dtype=torch.int32, device=scores.device)
    val = torch.empty((S, k), dtype=torch.float32, device=scores.device)
    a = L.TopkArgs()
    a.scores, a.num_segments, a.k, a.seg_len = scores.data_ptr(), S, k, N
    a.seg_stride = scores.stride(0) if S > 1 else N
    a.out_idx, a.out_val = idx.data_ptr(), val.data_ptr()
    need = L.lib().tka_topk_workspace_bytes(C.byref(a))
    ws = _workspace(need, scores.device)
    a.workspace, a.workspace_bytes, a.stream = ws.data_ptr(), ws.numel(), _stream()
    L.check(L.lib().tka_topk_f32(C.byref(a)), "tka_topk_f32")
    return idx, val


class CenterTopkPlan:
    """Argument block, outputs and workspace of one centre-only selection; run() is one C call."""

    def __init__(self, q, centers, top_c, cluster_len, scale=1.0):
        _need_cuda(q, centers)
        if not centers.is_contiguous() or not q.is_contiguous():
            raise ValueError("q and centers must be contiguous")
        H, Cn, _ = centers.shape
        self.q, self.centers = q, centers
        self.out = torch.empty((H, top_c * cluster_len), dtype=torch.int32, device=q.device)
        self.cen = torch.empty((H, top_c), dtype=torch.int32, device=q.device)
        self.val = torch.empty((H, top_c), dtype=torch.float32, device=q.device)
        a = self.args = L.CenterTopkArgs()
        a.q, a.centers, a.dtype = q.data_ptr(), centers.data_ptr(), _dtype_code(centers)
        a.num_heads, a.num_centers, a.top_c, a.cluster_len, a.head_dim = H, Cn, top_c, cluster_len, 128
        a.scale = scale
        a.out_idx, a.out_centers, a.out_center_val = self.out.data_ptr(), self.cen.data_ptr(), self.val.data_ptr()
        need = L.lib().tka_center_topk_expand_workspace_bytes(C.byref(a))
        self.ws = _own_workspace(need, q.device)
        a.workspace, a.workspace_bytes = self.ws.data_ptr(), self.ws.numel()

    def run(self):
        self.args.stream = _stream()
        L.check(L.lib().tka_center_topk_expand(C.byref(self.args)), "tka_center_topk_expand")
        return self


def center_topk_expand(q, centers, top_c, cluster_len, scale=1.0):
    """Centre-only selection.  q [H,128], centers [H,C,128] contiguous.
    Returns (token ids int32 [H, top_c*cluster_len], centre ids int32 [H,top_c], centre scores fp32 [H,top_c])."""
    plan = CenterTopkPlan(q, centers, top_c, cluster_len, scale).run()
    return plan.out, plan.cen, plan.val


def cluster_gemv_topk(q, centers, keys, top_c, cluster_len, k, scale=1.0):
    """Two-level selection.  q [H,128], centers [H,C,128], keys [C*cluster_len, H, 128].  Returns int32 [H, top_c*k]."""
    _need_cuda(q, centers, keys)
    H, Cn, _ = centers.shape
    out = torch.empty((H, top_c * k), dtype=torch.int32, device=q.device)
    a = L.ClusterTopkArgs()
    a.q, a.centers, a.keys, a.dtype = q.data_ptr(), centers.data_ptr(), keys.data_ptr(), _dtype_code(keys)
    a.num_heads, a.num_centers, a.top_c, a.cluster_len, a.k, a.head_dim = H, Cn, top_c, cluster_len, k, 128
    a.scale = scale
    a.key_stride_n, a.key_stride_h = keys.stride(0), keys.stride(1)
    a.out_idx = out.data_ptr()
    need = L.lib().tka_cluster_gemv_topk_workspace_bytes(C.byref(a))
    ws = _workspace(need, q.device)
    a.workspace, a.workspace_bytes, a.stream = ws.data_ptr(), ws.numel(), _stream()
    L.check(L.lib().tka_cluster_gemv_topk(C.byref(a)), "tka_cluster_gemv_topk")
    return out


def index_union(idx, sink, local, seq_len):
    """idx int32 [..., k] -> (union int32 [..., k+sink+local] ascending, -1 padded; count int32 [...])."""
    _need_cuda(idx)
    idx = idx.contiguous()
    k = idx.shape[-1]
    S = idx.numel() // k
    out = torch.empty(idx.shape[:-1] + (k + sink + local,), dtype=torch.int32, device=idx.device)
    cnt = torch.empty(idx.shape[:-1], dtype=torch.int32, device=idx.device)
    a = L.IndexUnionArgs()
    a.idx, a.num_segments, a.k, a.sink, a.local, a.seq_len = idx.data_ptr(), S, k, sink, local, seq_len
    a.out_idx, a.out_count, a.stream = out.data_ptr(), cnt.data_ptr(), _stream()
    L.check(L.lib().tka_index_union(C.byref(a)), "tka_index_union")
    return out, cnt


class FlashDecodePlan:
    """Argument block, output and workspace of one split-K decode configuration; run() is one C call."""

    def __init__(self, q, keys, values, scale, group=1, num_splits=0, kv_idx=None, kv_count=None, kv_logit=None,
                 out_dtype=None, return_lse=False, softmax_mode=L.TKA_SOFTMAX_SCALED):
        _need_cuda(q, keys, values, kv_idx, kv_count, kv_logit)
        q = _q3(q)
        B = q.shape[0]
        sb, sn, sh, N, H = _kv_strides(keys, B)
        if _kv_strides(values, B) != (sb, sn, sh, N, H):
            raise ValueError("keys and values must share shape and strides")
        out_dtype = out_dtype or q.dtype
        self.q, self.keys, self.values = q, keys, values
        self.out = torch.empty((B, H * group, 128), dtype=out_dtype, device=q.device)
        self.lse = torch.empty((B, H * group), dtype=torch.float32, device=q.device) if return_lse else None
        a = L.FlashDecodeArgs()
        a.q, a.keys, a.values, a.out = q.data_ptr(), keys.data_ptr(), values.data_ptr(), self.out.data_ptr()
        a.dtype, a.out_dtype = _dtype_code(keys), _DT[out_dtype]
        a.batch, a.num_kv_heads, a.group, a.head_dim = B, H, group, 128
        a.num_splits, a.softmax_mode = num_splits, softmax_mode
        a.seq_len, a.q_stride_b, a.out_stride_b = N, q.stride(0), self.out.stride(0)
        a.kv_stride_b, a.kv_stride_n, a.kv_stride_h = sb, sn, sh
        a.scale = scale
        if kv_idx is not None:
            self.kv_idx = kv_idx.contiguous()
            a.idx_len, a.kv_idx = self.kv_idx.shape[-1], self.kv_idx.data_ptr()
            if kv_count is not None:
                self.kv_count = kv_count.contiguous()
                a.kv_count = self.kv_count.data_ptr()
            if kv_logit is not None:
                self.kv_logit = kv_logit.contiguous()
                a.kv_logit = self.kv_logit.data_ptr()
        a.out_lse = self.lse.data_ptr() if self.lse is not None else None
        need = L.lib().tka_flash_decode_workspace_bytes(C.byref(a))
        self.ws = _own_workspace(need, q.device)
        a.workspace, a.workspace_bytes = self.ws.data_ptr(), self.ws.numel()
        self.args = a
        self._fn = L.lib().tka_flash_decode

    def run(self):
        self.args.stream = torch.cuda.current_stream().cuda_stream
        L.check(self._fn(C.byref(self.args)), "tka_flash_decode")
        return self


def flash_decode(q, keys, values, scale, group=1, num_splits=0, kv_idx=None, kv_count=None, kv_logit=None,
                 out_dtype=None, return_lse=False, softmax_mode=L.TKA_SOFTMAX_SCALED):
    """Split-K decode attention (dense, or over kv_idx [B,Hkv,L]).  Returns out [B,Hq,128] (and LSE fp32 [B,Hq])."""
    plan = FlashDecodePlan(q, keys, values, scale, group, num_splits, kv_idx, kv_count, kv_logit, out_dtype,
                           return_lse, softmax_mode).run()
    return (plan.out, plan.lse) if return_lse else plan.out


def lse_combine(part_m, part_l, part_acc, out_dtype=torch.float16, return_lse=False):
    """part_m, part_l fp32 [R,S]; part_acc fp32 [R,S,128] -> out [R,128]."""
    _need_cuda(part_m, part_l, part_acc)
    part_m, part_l, part_acc = part_m.contiguous(), part_l.contiguous(), part_acc.contiguous()
    R, S = part_m.shape
    out = torch.empty((R, 128), dtype=out_dtype, device=part_m.device)
    lse = torch.empty((R,), dtype=torch.float32, device=part_m.device) if return_lse else None
    a = L.LseCombineArgs()
    a.part_m, a.part_l, a.part_acc = part_m.data_ptr(), part_l.data_ptr(), part_acc.data_ptr()
    a.rows, a.num_splits, a.out_dtype = R, S, _DT[out_dtype]
    a.out = out.data_ptr()
    a.out_lse = lse.data_ptr() if lse is not None else None
    a.stream = _stream()
    L.check(L.lib().tka_lse_combine(C.byref(a)), "tka_lse_combine")
    return (out, lse) if return_lse else out


def retrieval_attention(q, k, v, out, topk, num_chunks=4, scale=1.0, softmax_mode=L.TKA_SOFTMAX_RAW_EXP,
                        bench_print=False, score_mode=L.TKA_SCORE_CANONICAL):
    """The reference op, general form: q [B,H,128], k/v [N,H,128] contiguous, writes out [B,H,128] in place."""
    _need_cuda(q, k, v, out)
    for t in (q, k, v, out):
        if not t.is_contiguous():
            raise ValueError("retrieval_attention expects contiguous tensors")
    if out.dtype != q.dtype or k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v, out must share one dtype")
    B, H, _ = q.shape
    a = L.RaArgs()
    a.q, a.keys, a.values, a.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.dtype, a.batch, a.num_heads, a.head_dim = _dtype_code(q), B, H, 128
    a.topk_per_chunk, a.num_chunks, a.softmax_mode, a.bench_print = topk, num_chunks, softmax_mode, int(bench_print)
    a.seq_len, a.scale, a.score_mode = k.shape[0], scale, score_mode
    need = L.lib().tka_retrieval_attention_workspace_bytes(C.byref(a))
    ws = _workspace(need, q.device)
    a.workspace, a.workspace_bytes, a.stream = ws.data_ptr(), ws.numel(), _stream()
    L.check(L.lib().tka_retrieval_attention(C.byref(a)), "tka_retrieval_attention")
    return out


class SparseDecodePlan:
    """Holds the argument block, outputs and workspace of one end-to-end decode configuration so that
    a step is a single C call (used by the benchmark and by callers that decode repeatedly)."""

    def __init__(self, q, keys, values, k, sink, local, scale, group, out_dtype=None, num_splits=0,
                 want_topk=True, want_union=True):
        _need_cuda(q, keys, values)
        q = _q3(q)
        B = q.shape[0]
        sb, sn, sh, N, H = _kv_strides(keys, B)
        if _kv_strides(values, B) != (sb, sn, sh, N, H):
            raise ValueError("keys and values must share shape and strides")
        out_dtype = out_dtype or q.dtype
        self.q, self.keys, self.values = q, keys, values
        self.out = torch.empty((B, H * group, 128), dtype=out_dtype, device=q.device)
        a = L.SparseDecodeArgs()
        a.q, a.keys, a.values, a.out = q.data_ptr(), keys.data_ptr(), values.data_ptr(), self.out.data_ptr()
        a.dtype, a.out_dtype = _dtype_code(keys), _DT[out_dtype]
        a.batch, a.num_kv_heads, a.group, a.head_dim = B, H, group, 128
        a.k, a.sink, a.local, a.num_splits = k, sink, local, num_splits
        a.seq_len, a.q_stride_b, a.out_stride_b = N, q.stride(0), self.out.stride(0)
        a.kv_stride_b, a.kv_stride_n, a.kv_stride_h = sb, sn, sh
        a.scale = scale
        self.topk_idx = self.topk_val = self.union_idx = self.union_count = None
        if want_topk:  # rank-ordered selection: costs a sort per KV head, not needed by the attention
            self.topk_idx = torch.empty((B, H, k), dtype=torch.int32, device=q.device)
            self.topk_val = torch.empty((B, H, k), dtype=torch.float32, device=q.device)
            a.out_topk_idx, a.out_topk_val = self.topk_idx.data_ptr(), self.topk_val.data_ptr()
        if want_union:
            self.union_idx = torch.empty((B, H, k + sink + local), dtype=torch.int32, device=q.device)
            self.union_count = torch.empty((B, H), dtype=torch.int32, device=q.device)
            a.out_union_idx, a.out_union_count = self.union_idx.data_ptr(), self.union_count.data_ptr()
        need = L.lib().tka_sparse_decode_workspace_bytes(C.byref(a))
        if need == 0:
            L.check(L.lib().tka_sparse_decode_step(C.byref(a)), "tka_sparse_decode_step")
        self.ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        a.workspace, a.workspace_bytes = self.ws.data_ptr(), self.ws.numel()
        self.args = a
        self._fn = L.lib().tka_sparse_decode_step

    def step(self):
        self.args.stream = torch.cuda.current_stream().cuda_stream
        rc = self._fn(C.byref(self.args))
        if rc != L.TKA_OK:
            L.check(rc, "tka_sparse_decode_step")
        return self.out

    def redone_segments(self):
        """Diagnostic: segments of the last step() that the selection kernel had to redo from the keys."""
        n = C.c_int32(0)
        L.check(L.lib().tka_sparse_decode_redone_segments(C.byref(self.args), C.byref(n)), "tka_sparse_decode_redone_segments")
        return n.value


def sparse_decode_step(q, keys, values, k, sink, local, scale, group, out_dtype=None, num_splits=0, want_topk=True):
    """End-to-end decode step.  Returns (out, topk_idx, topk_val, union_idx, union_count); without want_topk the
    rank-ordered selection is not produced (None)."""
    plan = SparseDecodePlan(q, keys, values, k, sink, local, scale, group, out_dtype, num_splits, want_topk=want_topk)
    plan.step()
    return plan.out, plan.topk_idx, plan.topk_val, plan.union_idx, plan.union_count


def set_test_hooks(force_segment_redo=0, tau_spin_limit=0, tau_withhold_mod=0, tau_withhold_rem=0, tau_withhold_mode=0,
                   union_handoff_order=0, fused_tail=0):
    """Testing hooks (see tka_test_hooks in include/topk_attn.h); no arguments = defaults."""
    h = L.TestHooks(force_segment_redo, tau_spin_limit, tau_withhold_mod, tau_withhold_rem, tau_withhold_mode, union_handoff_order,
                    fused_tail)
    L.check(L.lib().tka_set_test_hooks(C.byref(h)), "tka_set_test_hooks")


class ReadProbe:
    """A kernel that only reads a KV cache in the access pattern of the long-segment GEMV (`stream`) or of the gathered
    attention (`gather`, over idx [B,H,L]): what the memory system gives to that pattern (tka_probe_read)."""

    def __init__(self, keys, values=None, idx=None, threads=512, rounds=2, nontemporal=True, tokens_per_wg=256):
        _need_cuda(keys)
        B = keys.shape[0] if keys.dim() == 4 else 1
        sb, sn, sh, N, H = _kv_strides(keys, B)
        self.keep = (keys, values, idx)
        self.sink = torch.zeros(1, dtype=torch.int32, device=keys.device)
        a = L.ProbeArgs()
        a.keys, a.sink = keys.data_ptr(), self.sink.data_ptr()
        a.kind = L.TKA_PROBE_STREAM if idx is None else L.TKA_PROBE_GATHER
        a.batch, a.num_kv_heads, a.seq_len = B, H, N
        a.kv_stride_b, a.kv_stride_n, a.kv_stride_h = sb, sn, sh
        a.threads, a.rounds, a.nontemporal, a.tokens_per_wg = threads, rounds, int(nontemporal), tokens_per_wg
        if idx is not None:
            if values is None or _kv_strides(values, B) != (sb, sn, sh, N, H) or idx.dtype != torch.int32 or not idx.is_contiguous():
                raise ValueError("gather probe: values like keys, idx int32 [B,H,L] contiguous")
            a.values, a.idx, a.idx_len = values.data_ptr(), idx.data_ptr(), idx.shape[-1]
        self.args = a

    def run(self):
        self.args.stream = _stream()
        L.check(L.lib().tka_probe_read(C.byref(self.args)), "tka_probe_read")
        return self


def profile_enable(on=True):
    L.lib().tka_profile_enable(int(on))


def profile_reset():
    L.lib().tka_profile_reset()


def profile_read():
    """{kernel name: (total_ms, launches)} since the last reset (synchronises the recorded events)."""
    cap = 64
    names = (C.c_char_p * cap)()
    ms = (C.c_double * cap)()
    n_l = (C.c_int64 * cap)()
    n = L.lib().tka_profile_read(names, ms, n_l, cap)
    return {names[i].decode(): (ms[i], n_l[i]) for i in range(n)}
