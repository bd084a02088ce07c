"""Host mirror of the hot-path operators inside src/model.rs and src/deepseek.rs:
Q8Head, MlaCache + mla_attn_flash_q8_mqa, matvec_packed_nt, the MoE expert section."""
import ctypes as C

import numpy as np

from . import _lib, q8 as _q8
from ._lib import ACT_DS, ACT_SITU, ACT_SWIGLU, MODE_F32, MODE_Q8, ExpertTable, check, cur_stream, hptr, lib, ptr


class Q8Head:
    """model::Q8Head (src/model.rs:261-348) resident on the device.

    from_f32 / from_q8 take device tensors; matvec takes x [batch, cols] f32 on the device and returns logits
    [batch, rows].  scales_f16 selects the q8_0 storage form (f16 scales) or the reference's f32 scales."""

    def __init__(self, q, scales, rows, cols):
        self.q, self.scales, self.rows, self.cols = q, scales, rows, cols
        import torch
        self.scales_f16 = scales.dtype == torch.float16

    @staticmethod
    def from_f32(w, rows, cols, scales_f16=True):
        import torch
        if cols % 32 != 0:
            raise ValueError("q8 blocks are 32 wide")
        _lib.require_device()
        q = torch.empty((rows, cols), dtype=torch.int8, device=w.device)
        s = torch.empty((rows, cols // 32), dtype=torch.float16 if scales_f16 else torch.float32, device=w.device)
        check(lib.mk_dev_q8head_from_f32(ptr(w.contiguous()), rows, cols, ptr(q), ptr(s), int(scales_f16), cur_stream()))
        return Q8Head(q, s, rows, cols)

    @staticmethod
    def from_q8(q, scales, rows, cols):
        return Q8Head(q.contiguous(), scales.contiguous(), rows, cols)

    def matvec_q8(self, xq, out=None):
        """Rows against already-quantized activations (Q8Head::row_dot, src/model.rs:337-347)."""
        import torch
        batch = xq.q.numel() // self.cols
        if out is None:
            out = torch.empty((batch, self.rows), dtype=torch.float32, device=self.q.device)
        for b0 in range(0, batch, 8):
            nb = min(8, batch - b0)
            check(lib.mk_dev_q8_matvec(ptr(self.q), ptr(self.scales), int(self.scales_f16), self.rows, self.cols,
                                       C.c_void_p(xq.q.data_ptr() + b0 * self.cols), C.c_void_p(xq.scales.data_ptr() + b0 * (self.cols // 32) * 4),
                                       nb, C.c_void_p(out.data_ptr() + b0 * self.rows * 4), cur_stream()))
        return out

    def matvec(self, x, out=None):
        """Q8Head::matvec (src/model.rs:290-335): quantize x, integer block dots, f32 rescale."""
        _lib.require_device()
        x = x.contiguous().reshape(-1, self.cols)
        return self.matvec_q8(_q8.quantize_q8(x), out)

    def argmax(self, logits):
        """Greedy token per row, ties to the lowest index (src/model.rs:3271-3291)."""
        import torch
        batch, n = logits.shape
        ws = torch.empty(2 * batch * 1024, dtype=torch.float32, device=logits.device)
        idx = torch.empty(batch, dtype=torch.int32, device=logits.device)
        check(lib.mk_dev_argmax(ptr(logits.contiguous()), batch, n, ptr(ws), ptr(idx), cur_stream()))
        return idx


def matvec_packed_nt(packed, scales, rows, cols, x, m):
    """model::matvec_packed_nt (src/model.rs:2412-2447), exact f32: x [m, cols] (position-major) -> [m, rows]."""
    import torch
    _lib.require_device()
    out = torch.empty((m, rows), dtype=torch.float32, device=x.device)
    check(lib.mk_dev_mxfp4_matvec_nt(ptr(packed), ptr(scales), rows, cols, ptr(x.contiguous()), m, ptr(out), cur_stream()))
    return out


class MlaCache:
    """Shared-latent q8_0 MLA cache on the device (MlaCache, src/model.rs:765-781,1556-1618, in the absorbed form):
    per position L int8 + L/32 f16 scales (latent) and R int8 + R/32 f16 scales (decoupled rope key)."""

    def __init__(self, L, R, capacity, device="cuda"):
        import torch
        self.L, self.R, self.cap, self.n = L, R, capacity, 0
        self.lat_q = torch.zeros((capacity, L), dtype=torch.int8, device=device)
        self.lat_s = torch.zeros((capacity, L // 32), dtype=torch.float16, device=device)
        self.rope_q = torch.zeros((capacity, max(R, 1)), dtype=torch.int8, device=device)
        self.rope_s = torch.zeros((capacity, max(R // 32, 1)), dtype=torch.float16, device=device)
        self._ws = None

    def positions(self):
        return self.n

    def push(self, latent, rope):
        """MlaCache::push (src/model.rs:1583-1618): quantize one position at append."""
        if self.n >= self.cap:
            raise RuntimeError("MlaCache is full")
        _lib.require_device()
        check(lib.mk_dev_mla_cache_append(ptr(latent.contiguous()), ptr(rope.contiguous()), self.L, self.R, self.n, ptr(self.lat_q),
                                          ptr(self.lat_s), ptr(self.rope_q), ptr(self.rope_s), cur_stream()))
        self.n += 1

    def assign_q8(self, lat_q, lat_s, rope_q, rope_s):
        n = lat_q.shape[0]
        self.lat_q[:n], self.lat_s[:n], self.rope_q[:n, :self.R], self.rope_s[:n, :self.R // 32] = lat_q, lat_s, rope_q, rope_s
        self.n = n

    def to_f32(self):
        """MlaCache::to_f32 (src/model.rs:1623-1676): q * s."""
        n, L, R = self.n, self.L, self.R
        lat = (self.lat_q[:n].float().view(n, L // 32, 32) * self.lat_s[:n].float().unsqueeze(-1)).view(n, L)
        rope = (self.rope_q[:n, :R].float().view(n, R // 32, 32) * self.rope_s[:n, :R // 32].float().unsqueeze(-1)).view(n, R)
        return lat, rope


def mla_attn_flash_q8_mqa(cache, q, pos, scale, out=None):
    """model::mla_attn_flash_q8_mqa (src/model.rs:1804-1908) over the shared-latent cache: q [nh, L+R] f32 on the
    device, positions 0..=pos attended, returns [nh, L]."""
    import torch
    _lib.require_device()
    nh = q.shape[0]
    if q.shape[1] != cache.L + cache.R:
        raise ValueError("query width must be L + R")
    if pos >= cache.n:
        raise ValueError("pos is beyond the cached positions")
    need = lib.mk_mla_decode_workspace_bytes(nh, cache.L, pos + 1)
    if cache._ws is None or cache._ws.numel() < need:
        cache._ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    if out is None:
        out = torch.empty((nh, cache.L), dtype=torch.float32, device=q.device)
    check(lib.mk_dev_mla_q8_decode(ptr(cache.lat_q), ptr(cache.lat_s), ptr(cache.rope_q), ptr(cache.rope_s), pos, ptr(q.contiguous()), nh,
                                   cache.L, cache.R, float(scale), ptr(cache._ws), ptr(out), cur_stream()))
    return out


class MlaHeadsCache:
    """MlaCache in the reference's own layout (src/model.rs:765-781) on the device: per position and head a q8 K-nope
    row and a q8 V row (int8 + f32 scales), one shared f32 rope row.  push / assign_f32 / to_f32 / attention mirror
    MlaCache::push, ::assign_f32, ::to_f32 and mla_attn_flash_q8_mqa; attn with several queries is the attention loop
    of mla_prefill (src/model.rs:2080-2102)."""

    def __init__(self, nh, nope, rope, vd, capacity, device="cuda", hadamard=False):
        import torch
        self.nh, self.nope, self.rope, self.vd, self.cap, self.n = nh, nope, rope, vd, capacity, 0
        self.had = int(bool(hadamard))  # kv_hadamard (src/model.rs:1532-1535): takes effect when nope and vd are multiples of 64
        self.kq = torch.zeros((capacity, nh * nope), dtype=torch.int8, device=device)
        self.ks = torch.zeros((capacity, nh * nope // 32), dtype=torch.float32, device=device)
        self.kr = torch.zeros((capacity, rope), dtype=torch.float32, device=device)
        self.vq = torch.zeros((capacity, nh * vd), dtype=torch.int8, device=device)
        self.vs = torch.zeros((capacity, nh * vd // 32), dtype=torch.float32, device=device)
        self._ws = None

    def positions(self):
        return self.n

    def push(self, k_rows, v_rows):
        """k_rows [n_new, nh * (nope + rope)], v_rows [n_new, nh * vd] (or one row each) appended."""
        _lib.require_device()
        k_rows = k_rows.reshape(-1, self.nh * (self.nope + self.rope)).contiguous()
        v_rows = v_rows.reshape(-1, self.nh * self.vd).contiguous()
        n_new = k_rows.shape[0]
        if self.n + n_new > self.cap:
            raise RuntimeError("MlaCache is full")
        check(lib.mk_dev_mla_heads_append(ptr(k_rows), ptr(v_rows), n_new, self.nh, self.nope, self.rope, self.vd, self.n, self.had, ptr(self.kq),
                                          ptr(self.ks), ptr(self.kr), ptr(self.vq), ptr(self.vs), cur_stream()))
        self.n += n_new

    def assign_f32(self, k, v):
        """MlaCache::assign_f32 (src/model.rs:1680-1692): emptied, then refilled from f32 rows."""
        self.n = 0
        self.push(k, v)

    def to_f32(self):
        import torch
        _lib.require_device()
        k = torch.empty((self.n, self.nh * (self.nope + self.rope)), dtype=torch.float32, device=self.kq.device)
        v = torch.empty((self.n, self.nh * self.vd), dtype=torch.float32, device=self.kq.device)
        if self.n:
            check(lib.mk_dev_mla_heads_to_f32(ptr(self.kq), ptr(self.ks), ptr(self.kr), ptr(self.vq), ptr(self.vs), self.n, self.nh, self.nope,
                                              self.rope, self.vd, self.had, ptr(k), ptr(v), cur_stream()))
        return k, v

    def attn(self, q, pos0, scale):
        """q [m, nh * (nope + rope)]: query i attends the positions 0 ..= pos0 + i.  Returns [m, nh * vd]."""
        import torch
        _lib.require_device()
        q = q.reshape(-1, self.nh * (self.nope + self.rope)).contiguous()
        m = q.shape[0]
        if pos0 + m > self.n:
            raise ValueError("queries reach beyond the cached positions")
        need = lib.mk_mla_heads_workspace_bytes(m, self.nh, self.nope, self.vd)
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        out = torch.empty((m, self.nh * self.vd), dtype=torch.float32, device=q.device)
        check(lib.mk_dev_mla_heads_q8_attn(ptr(self.kq), ptr(self.ks), ptr(self.kr), ptr(self.vq), ptr(self.vs), pos0, ptr(q), m, self.nh,
                                           self.nope, self.rope, self.vd, float(scale), self.had, ptr(self._ws), ptr(out), cur_stream()))
        return out


class PackedExperts:
    """Expert table of an MoE layer on the device: per expert w1, w3 [inter, d] and w2 [d, inter], each MXFP4
    (packed, scales) in the reference layout, or -- a VQ1 expert (src/model.rs:729-730) -- (index bytes, None) with
    the file's 256 x 16 f32 `vq_codebook`.  Built from lists of device tensors.  pack: also keep every expert's matrices
    in the order the one-launch decode kernel streams them (mk_dev_moe_pack_gate_up / _down; as many bytes again), which
    lets up to 3 decode tokens take that kernel (calls on it must not overlap on one device); None = when the shapes are
    the ones it takes (d 7168 or 5120, inter 2048) and no expert is VQ1.  scales_by_tile: also keep every matrix's scale
    bytes in K-tile order (mk_dev_mxfp4_scales_by_tile; 1/16 of the experts' bytes again) for the matrix-core kernels of
    moe_decode from 4 tokens and of moe_prefill; None = when d and inter are multiples of 512 and no expert is VQ1."""

    def __init__(self, w1, w3, w2, d, inter, vq_codebook=None, pack=None, scales_by_tile=None):
        import torch
        self.d, self.inter, self.n = d, inter, len(w1)
        self._keep = (w1, w3, w2, vq_codebook)
        dev = w1[0][0].device
        arr = lambda lst, k: torch.tensor([t[k].data_ptr() if t[k] is not None else 0 for t in lst], dtype=torch.int64, device=dev)
        self._ptrs = [arr(w1, 0), arr(w1, 1), arr(w3, 0), arr(w3, 1), arr(w2, 0), arr(w2, 1)]
        self.has_vq = vq_codebook is not None
        any_vq = any(t[1] is None for lst in (w1, w3, w2) for t in lst)
        if any_vq and not self.has_vq:
            raise ValueError("a VQ1 expert needs the codebook")
        fits = not any_vq and d in (7168, 5120) and inter == 2048
        if pack is None:
            pack = fits
        self._pack, tptrs = None, [None, None]
        if pack:
            if not fits:
                raise ValueError("the packed copies need MXFP4 experts at d = 7168 or 5120 and inter = 2048")
            b13 = (lib.mk_moe_pack_bytes(d, inter, 0) + 255) // 256 * 256
            b2 = (lib.mk_moe_pack_bytes(d, inter, 1) + 255) // 256 * 256
            self._pack = torch.empty(self.n * (b13 + b2), dtype=torch.uint8, device=dev)
            base = self._pack.data_ptr()
            for i in range(self.n):
                at = base + i * (b13 + b2)
                check(lib.mk_dev_moe_pack_gate_up(ptr(w1[i][0]), ptr(w1[i][1]), ptr(w3[i][0]), ptr(w3[i][1]), d, inter, at, cur_stream()))
                check(lib.mk_dev_moe_pack_down(ptr(w2[i][0]), ptr(w2[i][1]), d, inter, at + b13, cur_stream()))
            self._tptrs = [torch.tensor([base + i * (b13 + b2) + k * b13 for i in range(self.n)], dtype=torch.int64, device=dev) for k in (0, 1)]
            tptrs = [p.data_ptr() for p in self._tptrs]
        # the scale bytes once more in K-tile order for the matrix-core kernels (None = when the shapes allow it)
        st_fits = not any_vq and d % 512 == 0 and inter % 512 == 0
        if scales_by_tile is None:
            scales_by_tile = st_fits
        stptrs = [None, None, None]
        if scales_by_tile:
            if not st_fits:
                raise ValueError("the K-tile ordered scale bytes need MXFP4 experts with d and inter multiples of 512")
            per = d * inter // 32
            self._st = torch.empty(self.n * 3 * per, dtype=torch.uint8, device=dev)
            base = self._st.data_ptr()
            for i in range(self.n):
                for k, (lst, r, c) in enumerate(((w1, inter, d), (w3, inter, d), (w2, d, inter))):
                    check(lib.mk_dev_mxfp4_scales_by_tile(ptr(lst[i][1]), r, c, base + (3 * i + k) * per, cur_stream()))
            self._stptrs = [torch.tensor([base + (3 * i + k) * per for i in range(self.n)], dtype=torch.int64, device=dev) for k in range(3)]
            stptrs = [p.data_ptr() for p in self._stptrs]
        self.table = ExpertTable(*[p.data_ptr() for p in self._ptrs], d, inter, self.n, vq_codebook.data_ptr() if self.has_vq else None, *tptrs,
                                 *stptrs)
        self._ws = None


def moe_decode(experts, ids, weights, x, shared=-1, mode=MODE_Q8, act_kind=ACT_SWIGLU, limit=0.0, out=None):
    """The expert section of moe_forward / ds_moe for B decode tokens in one grouped pass
    (src/model.rs:2227-2264,2346-2351; src/deepseek.rs:1069-1106).  ids [B, topk] int32, weights [B, topk] f32,
    x [B, d] f32, all on the device; returns [B, d]."""
    import torch
    _lib.require_device()
    B, topk = ids.shape
    need = _moe_ws_bytes(experts, B, topk, shared)
    if experts._ws is None or experts._ws.numel() < need:
        experts._ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    if out is None:
        out = torch.empty((B, experts.d), dtype=torch.float32, device=x.device)
    check(lib.mk_dev_moe_decode(C.byref(experts.table), B, topk, ptr(ids.contiguous()), ptr(weights.contiguous()), shared,
                                ptr(x.contiguous()), mode, act_kind, float(limit), ptr(experts._ws), ptr(out), cur_stream()))
    return out


def _moe_ws_bytes(experts, B, topk, shared):
    need = lib.mk_moe_decode_workspace_bytes(B, topk, int(shared >= 0), experts.d, experts.inter)
    if getattr(experts, "has_vq", False):
        need += lib.mk_moe_decode_vq_workspace_bytes(B, topk, int(shared >= 0), experts.d, experts.inter)
    return need


def _moe_ws(experts, B, topk, shared, device):
    import torch
    need = _moe_ws_bytes(experts, B, topk, shared)
    if experts._ws is None or experts._ws.numel() < need:
        experts._ws = torch.empty(need, dtype=torch.uint8, device=device)
    return experts._ws


def moe_decode_act(experts, ids, weights, x, shared=-1, mode=MODE_Q8, act_kind=ACT_SWIGLU, limit=0.0):
    """First half of moe_decode: ACT(W1_e x_t, W3_e x_t) per (token, slot) pair (the shared expert is the last slot),
    the f32 rows that the W2 matvec of src/model.rs:2255-2259 / src/deepseek.rs:1088-1089 takes.  Returns
    [B, per, inter]."""
    import torch
    _lib.require_device()
    B, topk = ids.shape
    per = topk + (1 if shared >= 0 else 0)
    act = torch.empty((B, per, experts.inter), dtype=torch.float32, device=x.device)
    check(lib.mk_dev_moe_decode_act(C.byref(experts.table), B, topk, ptr(ids.contiguous()), ptr(weights.contiguous()), shared,
                                    ptr(x.contiguous()), mode, act_kind, float(limit), ptr(_moe_ws(experts, B, topk, shared, x.device)),
                                    ptr(act), cur_stream()))
    return act


def moe_decode_from_act(experts, ids, weights, act, shared=-1, mode=MODE_Q8, act_kind=ACT_SWIGLU):
    """Second half of moe_decode: the W2 matvecs on given activation rows [B, per, inter] and the weighted sum in slot
    order (src/model.rs:2255-2259, 2346-2351).  Returns [B, d]."""
    import torch
    _lib.require_device()
    B, topk = ids.shape
    out = torch.empty((B, experts.d), dtype=torch.float32, device=act.device)
    check(lib.mk_dev_moe_decode_from_act(C.byref(experts.table), B, topk, ptr(ids.contiguous()), ptr(weights.contiguous()), shared,
                                         ptr(act.contiguous()), mode, act_kind, ptr(_moe_ws(experts, B, topk, shared, act.device)), ptr(out),
                                         cur_stream()))
    return out


def moe_prefill_intermediates(experts, T, topk):
    """Views of mk_dev_moe_prefill's intermediates inside the workspace of the last moe_prefill call on `experts`
    (grouping of src/model.rs:2539-2544 and the per-pair rows before the weighted sum): dict with order, pos,
    offsets (int32), g and u [P, inter] and o [P, d] (f32), rows in grouped order."""
    import torch
    lay = _lib.PrefillLayout()
    check(lib.mk_moe_prefill_workspace_layout(T, topk, experts.n, experts.d, experts.inter, C.byref(lay)))
    ws, P = experts._ws, T * topk
    i32 = lambda off, n: ws[off:off + 4 * n].view(torch.int32)
    f32 = lambda off, r, c: ws[off:off + 4 * r * c].view(torch.float32).view(r, c)
    return {"order": i32(lay.order, P), "pos": i32(lay.pos, P), "offsets": i32(lay.offsets, experts.n + 1),
            "g": f32(lay.g, P, experts.inter), "u": f32(lay.u, P, experts.inter), "o": f32(lay.o, P, experts.d)}


PREFILL_MAX_PAIRS = 16384  # (token, slot) pairs one mk_dev_moe_prefill* call takes


def moe_prefill(experts, ids, weights, x, act_kind=ACT_SWIGLU, out=None, keep=False, exact=False, bf16=False, mxfp8=False):
    """The expert section of moe_prefill (src/model.rs:2528-2602, 2690-2700) for T prompt positions: pairs grouped by
    expert, gate / up / activation / down per used expert, per-token weighted sum in slot order.  ids [T, topk] int32,
    weights [T, topk] f32, x [T, d] f32; returns [T, d].
    The arithmetic is the reference's own unless the caller asks for less (f32 rows and activation against the
    dequantized weights, f32 products and sums on the f32 matrix instruction: matvec_packed_nt per expert,
    src/model.rs:2580-2599; mk_dev_moe_prefill_f32; `exact=True` names the same thing).  The intermediates then hold
    ACT(gate, up) in "g", the up rows in "u" and the down rows in "o".
    bf16: hidden rows and activation rows rounded to bfloat16, exact weights, f32 products and sums on the bf16 matrix
    instruction (mk_dev_moe_prefill_bf16); "g" and "u" then hold the gate and up rows.
    mxfp8: activations as MXFP8 blocks on the block-scaled matrix cores (mk_dev_moe_prefill), the fastest form and the
    one with no counterpart in the reference: an explicit opt-in.  keep (mxfp8 only): also store the f32 gate and up
    rows (moe_prefill_intermediates reads them); the result is the same.
    A prompt of more than 16384 (token, slot) pairs is split into calls of whole tokens; the intermediates are then
    those of the last call."""
    import torch
    _lib.require_device()
    T, topk = ids.shape
    if bf16 + mxfp8 + exact > 1:
        raise ValueError("exact, bf16 and mxfp8 name three different arithmetics: pick one")
    if keep and not mxfp8:
        raise ValueError("keep belongs to the mxfp8 form (the others store their intermediates anyway)")
    step = max(1, PREFILL_MAX_PAIRS // topk)
    need = lib.mk_moe_prefill_workspace_bytes(min(T, step), topk, experts.n, experts.d, experts.inter)
    if experts._ws is None or experts._ws.numel() < need:
        experts._ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    if out is None:
        out = torch.empty((T, experts.d), dtype=torch.float32, device=x.device)
    fn = lib.mk_dev_moe_prefill_bf16 if bf16 else (lib.mk_dev_moe_prefill_keep if keep else lib.mk_dev_moe_prefill) if mxfp8 else lib.mk_dev_moe_prefill_f32
    ids, weights, x = ids.contiguous(), weights.contiguous(), x.contiguous()
    assert out.is_contiguous()
    for t0 in range(0, T, step):
        n = min(step, T - t0)
        check(fn(C.byref(experts.table), experts.n, n, topk, ptr(ids[t0:t0 + n]), ptr(weights[t0:t0 + n]), ptr(x[t0:t0 + n]), act_kind,
                 ptr(experts._ws), ptr(out[t0:t0 + n]), cur_stream()))
    return out


ROUTER_SOFTMAX, ROUTER_SIGMOID, ROUTER_SQRTSOFTPLUS = 0, 1, 2


def rmsnorm(x, w, eps, quantize=False):
    """model::rmsnorm / ds_rmsnorm (src/model.rs:599-605, src/deepseek.rs:241-248) for rows x [B, d] (or [d]) on the
    device, bit-identical to the reference.  With quantize=True also returns the q8 form of the normed rows
    (q [B, d] int8, scales [B, d/32] f32: q8::quantize_q8_into), the input of the q8-mode matvecs."""
    import torch
    _lib.require_device()
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    B, d = x2.shape
    out = torch.empty_like(x2)
    q = s = None
    if quantize:
        q = torch.empty((B, d), dtype=torch.int8, device=x.device)
        s = torch.empty((B, d // 32), dtype=torch.float32, device=x.device)
    check(lib.mk_dev_rmsnorm(ptr(x2), B, d, ptr(w.contiguous()), float(eps), ptr(out), ptr(q) if quantize else None,
                             ptr(s) if quantize else None, cur_stream()))
    out = out.reshape(x.shape)
    return (out, q, s) if quantize else out


def matvec(w, x):
    """model::matvec (src/model.rs:198-247): w [rows, cols] f32, x [cols] or [B, cols]; the reference's dot contract,
    bit-identical.  For the small f32 matrices of a layer (router gate, latent projections)."""
    import torch
    _lib.require_device()
    rows, cols = w.shape
    x2 = x.reshape(-1, cols).contiguous()
    out = torch.empty((x2.shape[0], rows), dtype=torch.float32, device=x.device)
    check(lib.mk_dev_matvec_f32(ptr(w.contiguous()), rows, cols, ptr(x2), x2.shape[0], ptr(out), cur_stream()))
    return out.reshape(x.shape[:-1] + (rows,))


def router_topk(logits, k, kind=ROUTER_SOFTMAX, bias=None, route_scale=1.0):
    """The reference's routing rules on logits [B, n]: softmax (benchmark layer), sigmoid + selection bias
    (src/model.rs:2151-2173), sqrt(softplus) + selection bias with route_scale (src/deepseek.rs:16-58)."""
    import torch
    _lib.require_device()
    B, n = logits.shape
    ids = torch.empty((B, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((B, k), dtype=torch.float32, device=logits.device)
    check(lib.mk_dev_router_topk(ptr(logits.contiguous()), B, n, k, kind, None if bias is None else ptr(bias.contiguous()),
                                 float(route_scale), ptr(ids), ptr(w), cur_stream()))
    return ids, w


def router_softmax_topk(logits, k):
    """Router of the benchmark MoE layer: softmax, top-k with the reference's tie rule, renormalised weights."""
    import torch
    _lib.require_device()
    B, n = logits.shape
    ids = torch.empty((B, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((B, k), dtype=torch.float32, device=logits.device)
    check(lib.mk_dev_router_softmax_topk(ptr(logits.contiguous()), B, n, k, ptr(ids), ptr(w), cur_stream()))
    return ids, w


def norm_gate_route(x, norm_w, eps, gate, k, kind=ROUTER_SOFTMAX, bias=None, route_scale=1.0, want_xn=True):
    """rmsnorm -> router gate matvec -> routing as one call of two launches (mk_dev_norm_gate_route): x [B, d], norm_w [d],
    gate [n, d].  Returns (xn [B, d] or None, logits [B, n], ids [B, k] int32, weights [B, k]), each bit-identical to
    rmsnorm, matvec and router_topk called one after the other."""
    import torch
    _lib.require_device()
    B, d = x.shape
    n = gate.shape[0]
    xn = torch.empty((B, d), dtype=torch.float32, device=x.device) if want_xn else None
    logits = torch.empty((B, n), dtype=torch.float32, device=x.device)
    ids = torch.empty((B, k), dtype=torch.int32, device=x.device)
    w = torch.empty((B, k), dtype=torch.float32, device=x.device)
    check(lib.mk_dev_norm_gate_route(ptr(x.contiguous()), B, d, ptr(norm_w.contiguous()), float(eps), ptr(gate.contiguous()), n, k, kind,
                                     None if bias is None else ptr(bias.contiguous()), float(route_scale), ptr(xn), ptr(logits), ptr(ids),
                                     ptr(w), cur_stream()))
    return xn, logits, ids, w


def grouped_gemm_f32(packed_list, scales_list, rows, cols, x, offsets, bf16=False):
    """matvec_packed_nt per group (src/model.rs:2412-2447 as called at src/model.rs:2580-2599): rows
    offsets[e]..offsets[e+1] of x [m, cols] against expert e -> [m, rows] f32.  x f32: the reference's f32 arithmetic on
    the f32 matrix instruction; bf16=True: x is a torch.bfloat16 tensor, exact weights, f32 products and sums on the
    bf16 matrix instruction."""
    import torch
    _lib.require_device()
    dev = x.device
    pp = torch.tensor([t.data_ptr() for t in packed_list], dtype=torch.int64, device=dev)
    sp = torch.tensor([t.data_ptr() for t in scales_list], dtype=torch.int64, device=dev)
    m = x.shape[0]
    assert x.is_contiguous() and x.dtype == (torch.bfloat16 if bf16 else torch.float32)
    out = torch.empty((m, rows), dtype=torch.float32, device=dev)
    fn = lib.mk_dev_mxfp4_grouped_gemm_bf16 if bf16 else lib.mk_dev_mxfp4_grouped_gemm_f32
    check(fn(ptr(pp), ptr(sp), len(packed_list), rows, cols, ptr(x), ptr(offsets), m, ptr(out), cur_stream()))
    return out


def grouped_gemm_split(packed_list, scales_list, rows, cols, codes, exps, offsets):
    """matvec_packed_nt per group (src/model.rs:2412-2447) on bfloat16-rounded rows given as two e4m3 terms per value
    (dequant.quantize_bf16_split), on the block-scaled matrix cores: rows offsets[e]..offsets[e+1] against expert e
    -> [m, rows] f32."""
    import torch
    _lib.require_device()
    dev = codes.device
    pp = torch.tensor([t.data_ptr() for t in packed_list], dtype=torch.int64, device=dev)
    sp = torch.tensor([t.data_ptr() for t in scales_list], dtype=torch.int64, device=dev)
    m = codes.shape[0]
    out = torch.empty((m, rows), dtype=torch.float32, device=dev)
    check(lib.mk_dev_mxfp4_grouped_gemm_split(ptr(pp), ptr(sp), len(packed_list), rows, cols, ptr(codes), ptr(exps), ptr(offsets), m, ptr(out),
                                              cur_stream()))
    return out


def grouped_gemm_mxfp8(packed_list, scales_list, rows, cols, codes, exps, offsets):
    """Per-expert batched evaluation of moe_prefill (src/model.rs:2539-2602) on the block-scaled matrix cores:
    rows offsets[e]..offsets[e+1] of the MXFP8 activations (codes, exps) against expert e -> [m, rows] f32."""
    import torch
    _lib.require_device()
    dev = codes.device
    pp = torch.tensor([t.data_ptr() for t in packed_list], dtype=torch.int64, device=dev)
    sp = torch.tensor([t.data_ptr() for t in scales_list], dtype=torch.int64, device=dev)
    m = codes.shape[0]
    out = torch.empty((m, rows), dtype=torch.float32, device=dev)
    check(lib.mk_dev_mxfp4_grouped_gemm(ptr(pp), ptr(sp), len(packed_list), rows, cols, ptr(codes), ptr(exps), ptr(offsets), m, ptr(out),
                                        cur_stream()))
    return out
