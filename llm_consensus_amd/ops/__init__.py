"""Functional op layer used by the models and the engine.

CUDA tensors (ROCm) go to the hand-written gfx950 kernels through ``ops.hip``; CPU
tensors go to the PyTorch oracles in ``ops.reference`` (plumbing/tests only). There is
no PyTorch fallback on the GPU path: if the kernel library is missing the call raises.
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import reference as ref

EPI_BF16, EPI_F32, EPI_SWIGLU = 0, 1, 2

# M at or below which the decode kernels (one activation panel) are used instead of the tile kernels.
WS_MAX_M = int(os.environ.get("LC_WS_MAX_M", "256"))
# Fewest 256x256 tiles for which the 256x256 pipelined kernel is used. It beats the 128x128 kernel
# even when its tiles cover a third of the CUs (160 tiles: 171 vs 308 us, 80 tiles: 145 vs 155 us at
# K = 8192), and below half coverage its split-K form takes over, so the default is "always".
# -1 disables the kernel (128x128 tiles everywhere).
GEMM256_MIN_TILES = int(os.environ.get("LC_GEMM256_MIN_TILES", "1"))
# Reduction depth from which prefill-sized GEMMs take the four-wave 256 x 256 kernel (gemm256w.hip):
# its longer prologue pays off only over many K-tiles (0 = never).
GEMM256W_MIN_K = int(os.environ.get("LC_GEMM256W_MIN_K", "8192")) or (1 << 30)
# Decode GEMM for 9..256 rows: the panel kernel (gemm_panel.hip, deep LDS-DMA ring) and its split-K policy.
PANEL_MAX_BLOCKS = int(os.environ.get("LC_PANEL_MAX_BLOCKS", "256"))
PANEL_MIN_KTILES = int(os.environ.get("LC_PANEL_MIN_KTILES", "4"))
# Ring depth of the panel kernel for M <= 128: deep (all of a CU's LDS, one workgroup per CU, fastest
# alone) or three stages (two workgroups per CU, for member engines that share the GPU on
# concurrent streams). Chosen when a decode graph is captured; see set_concurrent_engines().
PANEL_DEEP = os.environ.get("LC_PANEL_DEEP", "1") == "1"
PANEL_WIDE = os.environ.get("LC_PANEL_WIDE", "1") == "1"   # 160-column workgroups where they save a round (see linear())
PANEL_WIDE_MAX_M = int(os.environ.get("LC_PANEL_WIDE_MAX_M", "256"))


# Decode attention: how many of the KV splits the waves of one workgroup may take (1, 2 or 4).
ATTN_DECODE_MAX_WAVES = int(os.environ.get("LC_ATTN_WAVES", "4"))


def set_concurrent_engines(n: int) -> None:
    """Tells the op layer how many engines will issue decode steps on concurrent streams."""
    global PANEL_DEEP
    if "LC_PANEL_DEEP" not in os.environ:
        PANEL_DEEP = n <= 1
# In-workgroup K-split decode kernel (kgemm.hip): widest output it is used for, and a test override
# (-1 = automatic, 0 = never, 1/2/4 = force that many n-tiles per workgroup).
KGEMM_MAX_N = int(os.environ.get("LC_KGEMM_MAX_N", "8192"))
# Most rows the in-workgroup K-split kernel is used for. Measured against the panel kernel (with
# non-temporal weight loads) on HBM-resident weights: at 1 row it wins on the narrow projections
# (6144x4096 10.9 vs 13.0 us, 4096x4096 7.9 vs 9.3) and ties on the wide ones; at 8 rows it still wins
# those (11.9 vs 13.5, 8.4 vs 9.4) but loses where K is long (3584x18944: 26.5 vs 23.9); at 16 rows it
# loses everywhere (4096x14336: 28.3 vs 21.4, 3584x18944: 36.3 vs 24.2).
KGEMM_MAX_M = int(os.environ.get("LC_KGEMM_MAX_M", "8"))
KGEMM_LONG_K = 8192          # beyond this K the kernel is only used up to KGEMM_LONG_K_MAX_M rows
KGEMM_LONG_K_MAX_M = 4
KGEMM_FORCE_NTW = int(os.environ.get("LC_KGEMM_NTW", "-1"))


def _hip():
    from . import hip

    return hip


# ---------------------------------------------------------------------------- weights
def padded_rows(N: int) -> int:
    """Output rows are padded with zeros to whole column tiles: 256 (so the 256x256 prefill
    kernel and its split-K / grouped forms apply to every projection), 128 for tiny outputs."""
    return (N + 127) // 128 * 128 if N <= 128 else (N + 255) // 256 * 256


def pack_weight(W: torch.Tensor) -> torch.Tensor:
    """[N, K] row-major -> MFMA-fragment order [n_pad/16, K/32, 64, 8] (see gemm.hip):
    packed[nt, kt, lane, j] = W[nt*16 + (lane & 15), kt*32 + 8*(lane >> 4) + j]."""
    N, K = W.shape
    if K % 64:
        raise ValueError(f"K={K} must be a multiple of 64")
    n_pad = padded_rows(N)
    if n_pad != N:
        W = torch.cat([W, W.new_zeros(n_pad - N, K)], 0)
    return W.view(n_pad // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(n_pad // 16, K // 32, 64, 8)


def unpack_weight(Wp: torch.Tensor, N: int) -> torch.Tensor:
    nt, kt = Wp.shape[0], Wp.shape[1]
    return Wp.view(nt, kt, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nt * 16, kt * 32)[:N].contiguous()


def interleave_gate_up(Wg: torch.Tensor, Wu: torch.Tensor) -> torch.Tensor:
    """Row order for the fused SwiGLU epilogue: 16-row tiles alternate gate / up."""
    dff, K = Wg.shape
    if dff % 16:
        raise ValueError("d_ff must be a multiple of 16")
    return torch.stack([Wg.view(dff // 16, 16, K), Wu.view(dff // 16, 16, K)], 1).reshape(2 * dff, K)


@dataclass
class LinearWeight:
    """A linear layer's weights in device layout. ``data`` is packed on GPU and row-major
    [N, K] on CPU. ``swiglu`` marks gate/up interleaving (output width N/2)."""

    data: torch.Tensor
    n: int
    k: int
    bias: Optional[torch.Tensor] = None
    swiglu: bool = False

    @property
    def n_pad(self) -> int:
        return padded_rows(self.n)

    @property
    def is_packed(self) -> bool:
        return self.data.dim() == 4

    @classmethod
    def from_dense(cls, W: torch.Tensor, bias: Optional[torch.Tensor] = None, device=None, swiglu: bool = False,
                   dtype: torch.dtype = torch.bfloat16, any_shape: bool = False, plain: bool = False):
        """W row-major [N, K] in final row order (already interleaved when swiglu). With
        ``any_shape`` a weight the MFMA kernels do not take (fp32, or a reduction depth that is
        no multiple of 64) stays row-major on the GPU too and goes through the shape-agnostic
        kernel (hybrid.hip); without it such a weight is an error at the first product."""
        device = torch.device(device) if device is not None else W.device
        N, K = W.shape
        W = W.to(device=device, dtype=dtype)
        b = bias.to(device=device, dtype=dtype).contiguous() if bias is not None else None
        # ``plain``: row-major whatever the shape (small products whose input is an fp32 column slice)
        plain = plain or (any_shape and (dtype != torch.bfloat16 or K % 64 != 0))
        if plain and swiglu:
            raise ValueError("the shape-agnostic product has no SwiGLU epilogue")
        data = pack_weight(W) if (device.type == "cuda" and not plain) else W.contiguous()
        return cls(data, N, K, b, swiglu)

    def dense(self) -> torch.Tensor:
        return unpack_weight(self.data, self.n) if self.is_packed else self.data

    def nbytes(self) -> int:
        return self.data.numel() * self.data.element_size() + (self.bias.numel() * 2 if self.bias is not None else 0)


def _kgemm_ntw(n_pad: int, M: int, swiglu: bool, K: int = 0) -> int:
    """n-tiles per workgroup for the in-workgroup K-split kernel, or 0 to use another kernel.
    It re-reads the activations once per workgroup from L2, so it is limited to M <= 64 and
    to outputs narrow enough that this stays below the weight traffic."""
    if KGEMM_FORCE_NTW >= 0:
        return KGEMM_FORCE_NTW if M <= 64 else 0
    if M > KGEMM_MAX_M or n_pad > KGEMM_MAX_N or (K > KGEMM_LONG_K and M > KGEMM_LONG_K_MAX_M):
        return 0
    for ntw in (4, 2, 1):
        if swiglu and ntw < 2:
            break
        if n_pad // (16 * ntw) >= 256:
            return ntw
    return 2 if swiglu else 1


def _choose_panel_splits(n_pad: int, K: int) -> int:
    """K splits of the panel kernel (gemm_panel.hip). Its LDS ring admits one workgroup per CU,
    so the aim is as many workgroups as possible WITHOUT exceeding the 256 CUs (a 257th would
    run alone in a second round); every split is a whole number of 64-deep K-tiles and at
    least PANEL_MIN_KTILES of them."""
    blocks = n_pad // 128
    nk = K // 64
    best = 1
    for s in (2, 3, 4, 5, 6, 7, 8, 12, 14, 16):
        if blocks * s > PANEL_MAX_BLOCKS:
            break
        if nk % s == 0 and nk // s >= PANEL_MIN_KTILES:
            best = s
    return best


def _choose_gemm256_splits(tiles: int, K: int) -> int:
    """K splits for the 256x256 kernel when its tiles alone cover less than half of the CUs:
    the most splits that keep tiles * splits within the 256 CUs, in whole 64-deep K-tiles, at
    least 8 of them each (below that the pipeline's fill and the slab traffic dominate)."""
    if tiles * 2 > 256 or GEMM256_MAX_SPLITS <= 1:
        return 1
    nk = K // 64
    best = 1
    for s in (2, 3, 4, 6, 7, 8):
        if tiles * s > 256 or s > GEMM256_MAX_SPLITS:
            break
        if nk % s == 0 and nk // s >= 8:
            best = s
    return best


@dataclass
class PartialSum:
    """Un-reduced output of a split-K GEMM: ``part`` holds S fp32 slabs [S, M, N] whose sum
    (+ bias) is the product. Consumers that read the product exactly once (the residual-add
    RMSNorm, the RoPE/KV-write kernel) sum the slabs themselves, which removes one kernel
    launch per GEMM from the decode step; anything else calls ``reduce()``."""

    part: torch.Tensor
    bias: Optional[torch.Tensor] = None

    @property
    def shape(self):
        return self.part.shape[1:]

    def reduce(self, out_f32: bool = False) -> torch.Tensor:
        S, M, N = self.part.shape
        y = torch.empty(M, N, dtype=torch.float32 if out_f32 else torch.bfloat16, device=self.part.device)
        _hip().call("lc_splitk_reduce", self.part.data_ptr(), _hip().ptr(self.bias), y.data_ptr(), S, M, N, N,
                    1 if out_f32 else 0)
        return y


def use_four_wave_gemm(k: int, out_f32: bool = False) -> bool:
    """Whether a prefill-sized GEMM (256 x 256 tiles) of reduction depth ``k`` takes the four-wave
    kernel (gemm256w.hip) instead of the eight-wave one: from GEMM256W_MIN_K on (the down
    projections of the served models: K = 14336 / 18944 / 28672; QKV, O and gate/up have K = d_model).
    The four-wave kernel has bf16 and SwiGLU epilogues only and needs at least four K-tiles."""
    return not out_f32 and k >= max(GEMM256W_MIN_K, 256)


def use_wide_panel(M: int, n_pad: int, k: int) -> bool:
    """Whether a decode GEMM of ``M`` rows against ``n_pad`` columns takes the 160-column workgroups:
    its 128-column tiles would need a second round on the 256 CUs (and K is not split), while
    ten-n-tile workgroups cover it in one."""
    return (PANEL_WIDE and M <= PANEL_WIDE_MAX_M and n_pad // 128 > 256
            and (n_pad // 16 + 9) // 10 <= 256 and _choose_panel_splits(n_pad, k) == 1)


def linear(x: torch.Tensor, w: LinearWeight, out_f32: bool = False, defer_reduce: bool = False):
    """y = x @ W^T (+bias). With ``w.swiglu`` returns silu(gate)*up of width N/2. With
    ``defer_reduce`` a split-K product may come back as a ``PartialSum``."""
    M = x.shape[0]
    out_n = w.n // 2 if w.swiglu else w.n
    if not x.is_cuda:
        Wd = w.dense()
        y = ref.linear(x, Wd, w.bias, torch.float32)
        if w.swiglu:
            y = y.view(M, w.n // 32, 2, 16)
            y = (torch.nn.functional.silu(y[:, :, 0]) * y[:, :, 1]).reshape(M, out_n)
        return y if out_f32 else y.to(x.dtype)
    h = _hip()
    if not w.is_packed:
        if w.swiglu or w.data.dim() != 2:
            raise RuntimeError("GPU linear needs packed weights (LinearWeight.from_dense on a cuda device)")
        return linear_any(x, w, out_f32)
    if x.dtype != torch.bfloat16:
        raise TypeError(f"the MFMA products take bf16 activations, got {x.dtype}")
    x = x.contiguous()
    epi = EPI_SWIGLU if w.swiglu else (EPI_F32 if out_f32 else EPI_BF16)
    y = torch.empty(M, out_n, dtype=torch.float32 if (out_f32 and not w.swiglu) else torch.bfloat16, device=x.device)
    if M == 0:
        return y
    if M > WS_MAX_M:
        tiles256 = ((M + 255) // 256) * (w.n_pad // 256)
        # (the reduction of the split-K slabs works on whole groups of 32 columns)
        splits = _choose_gemm256_splits(tiles256, w.k) if (w.n_pad % 256 == 0 and not w.swiglu and w.n % 32 == 0) else 1
        if splits > 1 and GEMM256_MIN_TILES >= 0:
            # Too few 256x256 tiles to fill the chip (a few hundred rows, narrow output): split K.
            part = torch.empty(splits, M, w.n, dtype=torch.float32, device=x.device)
            h.call("lc_gemm256_splitk", w.data.data_ptr(), x.data_ptr(), part.data_ptr(), M, w.n, w.k, w.n_pad, w.n,
                   splits)
            if defer_reduce and not out_f32:
                return PartialSum(part, w.bias)
            h.call("lc_splitk_reduce", part.data_ptr(), h.ptr(w.bias), y.data_ptr(), splits, M, w.n, out_n,
                   1 if out_f32 else 0)
            return y
        if GEMM256_MIN_TILES >= 0 and w.n_pad % 256 == 0 and tiles256 >= GEMM256_MIN_TILES:
            # long K (down projections): four waves of 128 x 128 with the accumulators in AGPRs
            kern = "lc_gemm256w" if use_four_wave_gemm(w.k, epi == EPI_F32) else "lc_gemm256"
            h.call(kern, w.data.data_ptr(), x.data_ptr(), y.data_ptr(), h.ptr(w.bias), M, w.n, w.k, w.n_pad,
                   out_n, epi)
            return y
        h.call("lc_gemm_tile", w.data.data_ptr(), x.data_ptr(), y.data_ptr(), h.ptr(w.bias), M, w.n, w.k, w.n_pad,
               out_n, epi)
        return y
    # ---- decode shapes: one activation panel of at most 256 rows ----
    ntw = _kgemm_ntw(w.n_pad, M, w.swiglu, w.k)
    if ntw:   # a handful of rows, narrow output: K split over the waves of one workgroup
        h.call("lc_kgemm", w.data.data_ptr(), x.data_ptr(), y.data_ptr(), h.ptr(w.bias), M, w.n, w.k, w.n_pad,
               out_n, epi, ntw)
        return y
    # 257..320 column tiles of 128 (Qwen2.5-7B gate/up: 296): a second round would keep 40 CUs busy
    # as long as the first kept 256; workgroups of 160 columns cover the matrix in one round
    # (at 256 rows 85-88 us against 100 for the 256x256 tiles below on that matrix)
    wide = epi != EPI_F32 and use_wide_panel(M, w.n_pad, w.k)
    # 129..256 rows against more than 256 column tiles (vocabulary projection, very wide gate/up):
    # a second round of 128-column tiles would start; 256x256 tiles (half as many) do better.
    if M > 128 and not wide and w.n_pad // 128 > 256 and w.n_pad % 256 == 0 and GEMM256_MIN_TILES >= 0:
        h.call("lc_gemm256", w.data.data_ptr(), x.data_ptr(), y.data_ptr(), h.ptr(w.bias), M, w.n, w.k, w.n_pad,
               out_n, epi)
        return y
    kernel, splits, extra = "lc_gemm_panel", _choose_panel_splits(w.n_pad, w.k) if w.n % 32 == 0 else 1, (1 if PANEL_DEEP else 0,)
    if wide:
        extra = (2,)
    if splits == 1:
        h.call(kernel, w.data.data_ptr(), x.data_ptr(), y.data_ptr(), h.ptr(w.bias), M, w.n, w.k, w.n_pad, out_n, epi, 1,
               *extra)
        return y
    part = torch.empty(splits, M, w.n, dtype=torch.float32, device=x.device)
    h.call(kernel, w.data.data_ptr(), x.data_ptr(), part.data_ptr(), None, M, w.n, w.k, w.n_pad, w.n, EPI_F32, splits,
           *extra)
    if defer_reduce and not w.swiglu and not out_f32:
        return PartialSum(part, w.bias)
    mode = 2 if w.swiglu else (1 if out_f32 else 0)
    h.call("lc_splitk_reduce", part.data_ptr(), h.ptr(w.bias), y.data_ptr(), splits, M, w.n, out_n, mode)
    return y


# ---------------------------------------------------------------------------- elementwise
def embed(ids: torch.Tensor, E: torch.Tensor, feed: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> torch.Tensor:
    """x[t] = E[ids[t]]. ``feed`` = (tokens int32 [*], rows int32 [T]): row t with rows[t] >= 0
    takes the id tokens[rows[t]] instead (the token sampled by a row of the previous decode step,
    read on the device by a step that was launched before that step's results came back)."""
    if not ids.is_cuda:
        if feed is not None:
            tok, rows = feed
            ids = torch.where(rows >= 0, tok[rows.clamp_min(0).long()].to(ids.dtype), ids)
        return ref.embed(ids, E)
    h = _hip()
    T, d = ids.numel(), E.shape[1]
    x = torch.empty(T, d, dtype=E.dtype, device=E.device)
    h.call("lc_embed_gather", ids.data_ptr(), E.data_ptr(), x.data_ptr(), T, d, E.shape[0],
           feed[0].data_ptr() if feed is not None else None, feed[1].data_ptr() if feed is not None else None)
    return x


def rmsnorm(hstate: torch.Tensor, w: torch.Tensor, eps: float, delta=None) -> torch.Tensor:
    """y = RMSNorm(hstate [+ delta]) * w. When ``delta`` (a tensor or a ``PartialSum``) is
    given, ``hstate`` (the residual stream) is updated in place to hstate + delta first."""
    if not hstate.is_cuda:
        return ref.rmsnorm(hstate, w, eps, delta)
    h = _hip()
    T, d = hstate.shape
    y = torch.empty_like(hstate)
    if isinstance(delta, PartialSum) and delta.bias is not None:
        delta = delta.reduce()
    if isinstance(delta, PartialSum):
        h.call("lc_rmsnorm", hstate.data_ptr(), None, w.data_ptr(), y.data_ptr(), T, d, float(eps),
               delta.part.data_ptr(), delta.part.shape[0])
    else:
        h.call("lc_rmsnorm", hstate.data_ptr(), h.ptr(delta), w.data_ptr(), y.data_ptr(), T, d, float(eps), None, 0)
    return y


def embed_pool(hidden: torch.Tensor, cu: torch.Tensor, mode: int = 0) -> torch.Tensor:
    """Pooled, L2-normalised embeddings of the sequences whose rows are [cu[s], cu[s+1])
    (mode 0: mean, 1: last row)."""
    return embed_pool_ranges(hidden, cu[:-1], cu[1:], mode)


def embed_pool_ranges(hidden: torch.Tensor, begin: torch.Tensor, end: torch.Tensor, mode: int = 0) -> torch.Tensor:
    """As ``embed_pool`` over explicit row ranges; mode 2 returns the plain fp32 row sums
    (chunked prompts add their chunk sums and normalise at the end with ``l2_normalize``)."""
    if not hidden.is_cuda:
        if mode == 2:
            return torch.stack([hidden[int(b):int(e)].float().sum(0) for b, e in zip(begin, end)])
        return torch.stack([ref.embed_pool(hidden, torch.tensor([int(b), int(e)]), mode)[0] for b, e in zip(begin, end)])
    h = _hip()
    n = begin.numel()
    begin, end = begin.contiguous(), end.contiguous()
    out = torch.empty(n, hidden.shape[1], dtype=torch.float32, device=hidden.device)
    h.call("lc_embed_pool", hidden.data_ptr(), begin.data_ptr(), end.data_ptr(), out.data_ptr(), n, hidden.shape[1], mode)
    return out


def l2_normalize(x: torch.Tensor) -> torch.Tensor:
    """Rows of fp32 ``x`` scaled to unit length (zero rows stay zero)."""
    if not x.is_cuda:
        return x / x.norm(dim=-1, keepdim=True).clamp_min(1e-30)
    h = _hip()
    x = x.contiguous()
    y = torch.empty_like(x)
    h.call("lc_l2_normalize", x.data_ptr(), y.data_ptr(), x.shape[0], x.shape[1])
    return y


# ---------------------------------------------------------------------------- rope + cache
def rope_kv_write(qkv, positions, slot_mapping, cos_t, sin_t, k_cache, vt_cache, Hq, Hkv, Dh) -> torch.Tensor:
    """Rotates Q in place and writes rotated K / V into the paged cache. ``qkv`` may be a
    ``PartialSum``; returns the bf16 [T, (Hq+2Hkv)*Dh] buffer whose Q section attention reads."""
    if isinstance(qkv, PartialSum):
        h = _hip()
        S, T, N = qkv.part.shape
        out = torch.empty(T, N, dtype=torch.bfloat16, device=qkv.part.device)
        h.call("lc_rope_kv_write", out.data_ptr(), positions.data_ptr(), slot_mapping.data_ptr(), cos_t.data_ptr(),
               sin_t.data_ptr(), k_cache.data_ptr(), vt_cache.data_ptr(), T, Hq, Hkv, Dh, k_cache.shape[2],
               cos_t.shape[0], qkv.part.data_ptr(), S, h.ptr(qkv.bias))
        return out
    if not qkv.is_cuda:
        ref.rope_kv_write(qkv, positions, slot_mapping, cos_t, sin_t, k_cache, vt_cache, Hq, Hkv, Dh)
        return qkv
    h = _hip()
    h.call("lc_rope_kv_write", qkv.data_ptr(), positions.data_ptr(), slot_mapping.data_ptr(), cos_t.data_ptr(),
           sin_t.data_ptr(), k_cache.data_ptr(), vt_cache.data_ptr(), qkv.shape[0], Hq, Hkv, Dh, k_cache.shape[2],
           cos_t.shape[0], None, 0, None)
    return qkv


def copy_blocks(kv_base: torch.Tensor, src: torch.Tensor, dst: torch.Tensor, block_elems: int, n_planes: int,
                plane_elems: int) -> None:
    """kv_base is the flat KV pool; planes (layer x {K,V}) are plane_elems apart."""
    if not kv_base.is_cuda:
        flat = kv_base.view(n_planes, plane_elems // block_elems, block_elems)
        flat[:, dst.long()] = flat[:, src.long()]
        return
    h = _hip()
    es = kv_base.element_size()
    h.call("lc_copy_blocks", kv_base.data_ptr(), src.data_ptr(), dst.data_ptr(), src.numel(), block_elems * es,
           plane_elems * es, n_planes)


# ---------------------------------------------------------------------------- attention
def attn_prefill(qkv, k_cache, vt_cache, block_tables, cu_q, ctx_lens, max_q_len, Hq, Hkv, Dh, scale,
                 window: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """qkv [T, (Hq+2Hkv)*Dh] after rope_kv_write; returns [T, Hq*Dh] (written into ``out``, a
    contiguous row range of a larger tensor, when given)."""
    T = qkv.shape[0]
    if not qkv.is_cuda:
        r = ref.attn_prefill(qkv[:, : Hq * Dh], k_cache, vt_cache, block_tables, cu_q, ctx_lens, Hq, Hkv, Dh,
                             scale, window)
        return r if out is None else out.copy_(r)
    h = _hip()
    if out is None:
        out = torch.empty(T, Hq * Dh, dtype=qkv.dtype, device=qkv.device)
    h.call("lc_attn_prefill", qkv.data_ptr(), qkv.stride(0), k_cache.data_ptr(), vt_cache.data_ptr(),
           block_tables.data_ptr(), block_tables.shape[1], cu_q.data_ptr(), ctx_lens.data_ptr(), out.data_ptr(),
           ctx_lens.numel(), int(max_q_len), Hq, Hkv, Dh, k_cache.shape[2], float(scale), int(window))
    return out


MOE_PANEL_MAX_ROWS = int(os.environ.get("LC_MOE_PANEL_ROWS", "640"))   # routed rows (tokens x top-k) up to which the MoE GEMMs use the panel kernel
MOE_GEMM256_MIN_ROWS = int(os.environ.get("LC_MOE_G256_ROWS", "641"))   # routed rows from which the 256x256 grouped GEMM is used
GEMM256_MAX_SPLITS = int(os.environ.get("LC_G256_SPLITS", "8"))
ATTN_PREFIX_WAVES = 4   # 1 = one wave per prefix piece and one partial slot per piece
# The per-row pass folds the shared-prefix partials in and writes the final rows (LC_ATTN_FOLD_PREFIX=0:
# the three-launch form with a separate merge, kept for comparison runs).
ATTN_FOLD_PREFIX = os.environ.get("LC_ATTN_FOLD_PREFIX", "1") == "1"


def choose_kv_splits(B: int, Hkv: int, max_ctx: int) -> int:
    """KV splits per (sequence, kv head): about 1024 waves in total (4 per CU) without slicing
    below 128 keys. Measured with an HBM-resident cache (benchmarks/attn_decode_bench.py): fewer
    waves leave the memory pipe short of requests, more waves shorten every wave's key loop
    until its fixed cost (query load, block-table walk, merge) dominates: 64 sequences x 8 kv
    heads x 544 keys run at 3.0 / 4.2 / 3.7 / 2.7 TB/s with 1 / 2 / 4 / 8 splits."""
    waves = max(1, B * Hkv)
    want = max(1, 1024 // waves)
    cap = max(1, max_ctx // 128)
    return int(max(1, min(want, cap, 16)))


def attn_decode(qkv, k_cache, vt_cache, block_tables, ctx_lens, Hq, Hkv, Dh, scale, window: int = 0,
                nsplit: int = 1, groups: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None,
                kv_begin: Optional[torch.Tensor] = None, max_group_rows: int = 0,
                prefix_splits: int = 1, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One query token per row of qkv [B, (Hq+2Hkv)*Dh]. ``groups`` = (first, count,
    shared_blocks) int32 device tensors enables the shared-prefix pass: rows of a group
    attend to their common leading blocks in one MFMA pass and ``kv_begin`` [B] tells the
    per-row pass where each row's private suffix starts."""
    B = qkv.shape[0]
    if not qkv.is_cuda:
        r = ref.attn_decode(qkv[:, : Hq * Dh], k_cache, vt_cache, block_tables, ctx_lens, Hq, Hkv, Dh, scale,
                            window)
        return r if out is None else out.copy_(r)
    h = _hip()
    if out is None:
        out = torch.empty(B, Hq * Dh, dtype=qkv.dtype, device=qkv.device)
    use_prefix = groups is not None and max_group_rows > 1
    # Up to four of the requested KV splits are taken by the waves of one workgroup, which
    # merges them on chip; only the remaining factor produces partial slots in HBM.
    waves = (4 if nsplit >= 4 else (2 if nsplit >= 2 else 1)) if Hq // Hkv <= 8 else 1
    waves = min(waves, ATTN_DECODE_MAX_WAVES)
    nsplit = max(1, nsplit // waves)
    if nsplit == 1 and not use_prefix:
        h.call("lc_attn_decode", qkv.data_ptr(), qkv.stride(0), k_cache.data_ptr(), vt_cache.data_ptr(),
               block_tables.data_ptr(), block_tables.shape[1], ctx_lens.data_ptr(), None, out.data_ptr(), None, None,
               1, 1, B, Hq, Hkv, Dh, k_cache.shape[2], float(scale), int(window), waves, 0)
        return out
    # The prefix pass merges four pieces of its key range on chip the same way.
    pwaves = 4 if (use_prefix and prefix_splits >= 4 and ATTN_PREFIX_WAVES >= 4) else 1
    prefix_splits = max(1, prefix_splits // pwaves)
    np_total = nsplit + (prefix_splits if use_prefix else 0)
    part_o = torch.empty(B, Hq, np_total, Dh, dtype=torch.float32, device=qkv.device)
    part_lse = torch.empty(B, Hq, np_total, dtype=torch.float32, device=qkv.device)
    # With one private split per row the per-row pass runs AFTER the shared-prefix pass and folds
    # the prefix slots into its own result: two launches and no partial slot for the private range
    # (16 x 16-chain step of Llama-3-8B: 7.70 -> 7.61 ms; both passes as one launch of independent
    # workgroups + merge measured 7.72: they do not overlap, the per-row pass is bound by its ~30 MB of private keys).
    fold = use_prefix and nsplit == 1 and waves == 1 and kv_begin is not None and ATTN_FOLD_PREFIX
    if use_prefix and fold:
        gf, gc, gs = groups
        h.call("lc_attn_prefix", qkv.data_ptr(), qkv.stride(0), k_cache.data_ptr(), vt_cache.data_ptr(),
               block_tables.data_ptr(), block_tables.shape[1], gf.data_ptr(), gc.data_ptr(), gs.data_ptr(),
               gf.numel(), int(max_group_rows), int(prefix_splits), part_o.data_ptr(), part_lse.data_ptr(), np_total,
               nsplit, Hq, Hkv, Dh, k_cache.shape[2], float(scale), pwaves)
    h.call("lc_attn_decode", qkv.data_ptr(), qkv.stride(0), k_cache.data_ptr(), vt_cache.data_ptr(),
           block_tables.data_ptr(), block_tables.shape[1], ctx_lens.data_ptr(),
           kv_begin.data_ptr() if (use_prefix and kv_begin is not None) else None, out.data_ptr(), part_o.data_ptr(),
           part_lse.data_ptr(), np_total, nsplit, B, Hq, Hkv, Dh, k_cache.shape[2], float(scale), int(window), waves,
           1 if fold else 0)
    if fold:
        return out
    if use_prefix:
        gf, gc, gs = groups
        h.call("lc_attn_prefix", qkv.data_ptr(), qkv.stride(0), k_cache.data_ptr(), vt_cache.data_ptr(),
               block_tables.data_ptr(), block_tables.shape[1], gf.data_ptr(), gc.data_ptr(), gs.data_ptr(),
               gf.numel(), int(max_group_rows), int(prefix_splits), part_o.data_ptr(), part_lse.data_ptr(), np_total,
               nsplit, Hq, Hkv, Dh, k_cache.shape[2], float(scale), pwaves)
    h.call("lc_attn_merge", part_o.data_ptr(), part_lse.data_ptr(), out.data_ptr(), np_total, B * Hq, Dh)
    return out


# ---------------------------------------------------------------------------- sampling
def sample(logits, temperature, top_p, top_k, seeds, steps, row_index=None, out_tok: Optional[torch.Tensor] = None):
    """logits fp32 [*, V]; per-row params are device tensors (float32/float32/int32/int64/int32).
    Returns (tokens int32 [R], logprobs float32 [R]); the tokens are written into ``out_tok``
    (int32, at least R long) when given."""
    if not logits.is_cuda:
        tok, lp = ref.sample(logits, temperature, top_p, top_k, seeds, steps, row_index)
        if out_tok is not None:
            out_tok[: tok.numel()].copy_(tok)
            tok = out_tok[: tok.numel()]
        return tok, lp
    h = _hip()
    R = temperature.numel()
    tok = out_tok[:R] if out_tok is not None else torch.empty(R, dtype=torch.int32, device=logits.device)
    lp = torch.empty(R, dtype=torch.float32, device=logits.device)
    h.call("lc_sample", logits.data_ptr(), logits.shape[1], logits.stride(0), h.ptr(row_index),
           temperature.data_ptr(), h.ptr(top_p), h.ptr(top_k), seeds.data_ptr(), h.ptr(steps), tok.data_ptr(),
           lp.data_ptr(), R)
    return tok, lp


def logprob_gather(logits, ids, row_index=None) -> torch.Tensor:
    """log_softmax(logits[row])[ids]. ids int32 [C] (shared) or [R, C]."""
    if not logits.is_cuda:
        return ref.logprob_gather(logits, ids, row_index)
    h = _hip()
    R = row_index.numel() if row_index is not None else logits.shape[0]
    C = ids.shape[-1]
    out = torch.empty(R, C, dtype=torch.float32, device=logits.device)
    h.call("lc_logprob_gather", logits.data_ptr(), logits.shape[1], logits.stride(0), h.ptr(row_index),
           ids.data_ptr(), C if ids.dim() == 2 else 0, C, out.data_ptr(), R)
    return out


def logit_targets_shard(logits, ids, vocab_lo: int, row_index=None) -> torch.Tensor:
    """One vocabulary shard's share of ``logprob_gather``: fp32 [R, Cp] with the raw logits of the
    targets that fall into columns [vocab_lo, vocab_lo + V_local) (0 elsewhere) in columns
    [0, C), the shard's log-sum-exp in column C and zero padding up to Cp = C + 1 rounded up to
    four floats (whole 16-byte rows for the exchange). ``logprob_merge`` combines the shards."""
    C = ids.shape[-1]
    Cp = (C + 1 + 3) // 4 * 4
    R = row_index.numel() if row_index is not None else logits.shape[0]
    if not logits.is_cuda:
        rows = logits[row_index.long()] if row_index is not None else logits
        local = ids.long() - vocab_lo
        local = local.expand(R, C) if local.dim() == 2 else local.view(1, C).expand(R, C)
        mine = (local >= 0) & (local < rows.shape[1])
        out = torch.zeros(R, Cp, dtype=torch.float32)
        out[:, :C] = torch.where(mine, rows.gather(1, local.clamp(0, rows.shape[1] - 1)), torch.zeros(()))
        out[:, C] = torch.logsumexp(rows.float(), dim=-1)
        return out
    h = _hip()
    out = torch.empty(R, Cp, dtype=torch.float32, device=logits.device)
    h.call("lc_logit_targets_shard", logits.data_ptr(), logits.shape[1], logits.stride(0), h.ptr(row_index),
           ids.data_ptr(), C if ids.dim() == 2 else 0, C, Cp, int(vocab_lo), out.data_ptr(), R)
    return out


def logprob_merge(parts: torch.Tensor, C: int) -> torch.Tensor:
    """parts fp32 [W, R, Cp] (``logit_targets_shard`` of W vocabulary shards) -> log-softmax values
    of the targets, fp32 [R, C]."""
    W, R, Cp = parts.shape
    if not parts.is_cuda:
        return parts[:, :, :C].sum(0) - torch.logsumexp(parts[:, :, C], dim=0).unsqueeze(1)
    h = _hip()
    parts = parts.contiguous()
    out = torch.empty(R, C, dtype=torch.float32, device=parts.device)
    h.call("lc_logprob_merge", parts.data_ptr(), W, R, C, Cp, out.data_ptr())
    return out


def zero_(t: torch.Tensor) -> torch.Tensor:
    """Fills a contiguous tensor whose size is a multiple of 4 bytes with zero bits (in place)."""
    if not t.is_cuda:
        return t.zero_()
    nbytes = t.numel() * t.element_size()
    if nbytes % 4 or not t.is_contiguous():
        raise ValueError("zero_ needs a contiguous tensor of a multiple of 4 bytes")
    if nbytes:
        _hip().call("lc_fill_f32", t.data_ptr(), 0.0, nbytes // 4)
    return t


def accumulate_(y: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """y += x for fp32 tensors of one shape (in place)."""
    if not y.is_cuda:
        return y.add_(x)
    h = _hip()
    h.call("lc_accumulate_f32", y.data_ptr(), x.contiguous().data_ptr(), y.numel())
    return y


def pad_cols(x: torch.Tensor, n_pad: int, fill: float) -> torch.Tensor:
    """fp32 [R, n] -> [R, n_pad] with ``fill`` in the new columns."""
    R, n = x.shape
    if n == n_pad:
        return x
    if not x.is_cuda:
        return torch.nn.functional.pad(x, (0, n_pad - n), value=fill)
    h = _hip()
    out = torch.empty(R, n_pad, dtype=torch.float32, device=x.device)
    h.call("lc_pad_cols_f32", x.contiguous().data_ptr(), out.data_ptr(), R, n, n_pad, float(fill))
    return out


def concat_cols(parts: torch.Tensor, total_cols: Optional[int] = None) -> torch.Tensor:
    """[W, R, c] -> [R, W * c] (the W blocks side by side), cut to ``total_cols`` columns."""
    W, R, c = parts.shape
    total = W * c if total_cols is None else int(total_cols)
    if not parts.is_cuda:
        return parts.permute(1, 0, 2).reshape(R, W * c)[:, :total]
    es = parts.element_size()
    if es % 2:
        raise ValueError("concat_cols needs elements of 2 or 4 bytes")
    h = _hip()
    parts = parts.contiguous()
    out = torch.empty(R, total, dtype=parts.dtype, device=parts.device)
    u = es // 2
    h.call("lc_concat_cols", parts.data_ptr(), W, R, c * u, total * u, out.data_ptr())
    return out


def gather_rows(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """x[rows] for a bf16 matrix and int32 row numbers (the embedding-gather kernel: a row
    gather is what it is)."""
    if not x.is_cuda:
        return x[rows.long()]
    if x.dtype == torch.float32:           # the fp32 residual stream of the hybrid decoders
        return embed_rows(rows, x.contiguous(), None)[0]
    return embed(rows, x)


# ---------------------------------------------------------------------------- MoE
@dataclass
class ExpertWeights:
    """Stacked per-expert weights. GPU: packed [E, n_pad/16, K/32, 64, 8]; CPU: [E, N, K]."""

    data: torch.Tensor
    n: int
    k: int
    swiglu: bool = False

    @property
    def n_pad(self) -> int:
        return padded_rows(self.n)

    @classmethod
    def from_dense(cls, W: torch.Tensor, device=None, swiglu: bool = False):
        device = torch.device(device) if device is not None else W.device
        E, N, K = W.shape
        W = W.to(device=device, dtype=torch.bfloat16)
        data = torch.stack([pack_weight(W[e]) for e in range(E)]) if device.type == "cuda" else W.contiguous()
        return cls(data, N, K, swiglu)

    def nbytes(self) -> int:
        return self.data.numel() * self.data.element_size()


def moe_route(x: torch.Tensor, Wr: torch.Tensor, topk: int):
    """Top-k routing with softmax over the selected logits: (ids int32 [T,k], weights fp32 [T,k])."""
    if not x.is_cuda:
        ids, wts, _ = ref.moe_router(x, Wr, topk)
        return ids.to(torch.int32), wts
    h = _hip()
    T, d = x.shape
    ids = torch.empty(T, topk, dtype=torch.int32, device=x.device)
    wts = torch.empty(T, topk, dtype=torch.float32, device=x.device)
    h.call("lc_moe_router", x.data_ptr(), Wr.data_ptr(), T, d, Wr.shape[0], topk, ids.data_ptr(), wts.data_ptr(), None)
    return ids, wts


def _expert_mlp_cpu(xe: torch.Tensor, w_gate_up: "ExpertWeights", w_down: "ExpertWeights", e: int) -> torch.Tensor:
    gu = ref.linear(xe, w_gate_up.data[e], None, torch.float32)
    gu = gu.view(-1, w_gate_up.n // 32, 2, 16)
    act = (torch.nn.functional.silu(gu[:, :, 0]) * gu[:, :, 1]).reshape(xe.shape[0], -1).to(xe.dtype)
    return ref.linear(act, w_down.data[e], None, xe.dtype).float()


def moe_permute(ids: torch.Tensor, E: int):
    """Sorts the (token, k) pairs of ``ids`` [T, k] by expert, keeping token order inside an
    expert. Returns (offsets int32 [E+1], sorted_src int32 [T*k]: token row of every sorted
    position, slot_of int32 [T*k]: sorted position of pair t*k + j)."""
    T, topk = ids.shape
    A = T * topk
    dev = ids.device
    if not ids.is_cuda:
        flat = ids.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        counts = torch.bincount(flat, minlength=E)
        offsets = torch.zeros(E + 1, dtype=torch.int32)
        offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
        slot_of = torch.empty(A, dtype=torch.int32)
        slot_of[order] = torch.arange(A, dtype=torch.int32)
        return offsets, (order // topk).to(torch.int32), slot_of
    h = _hip()
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    sorted_src = torch.empty(A, dtype=torch.int32, device=dev)
    slot_of = torch.empty(A, dtype=torch.int32, device=dev)
    h.call("lc_moe_permute", ids.data_ptr(), T, topk, E, offsets.data_ptr(), sorted_src.data_ptr(), slot_of.data_ptr())
    return offsets, sorted_src, slot_of


def experts_on_sorted(x: torch.Tensor, row_index: Optional[torch.Tensor], offsets: torch.Tensor, expert0: int,
                      w_gate_up: "ExpertWeights", w_down: "ExpertWeights", rows_bound: int,
                      zero_unwritten: bool = False) -> torch.Tensor:
    """The resident experts' SwiGLU MLPs over rows in expert-sorted order. Sorted position p
    in [offsets[expert0 + e], offsets[expert0 + e + 1]) belongs to resident expert e and reads
    ``x[row_index[p]]``. Returns y [rows_bound, d]; positions outside the resident experts'
    ranges are left unwritten (zero with ``zero_unwritten``). ``rows_bound`` (a host integer)
    bounds every offset, so nothing here waits for the device."""
    E_local = w_gate_up.data.shape[0]
    d = w_down.n
    dff = w_gate_up.n // 2
    dev = x.device
    if not x.is_cuda:
        y = torch.zeros(rows_bound, d, dtype=x.dtype)
        for e in range(E_local):
            lo, hi = int(offsets[expert0 + e]), int(offsets[expert0 + e + 1])
            if hi > lo:
                rows = x[row_index[lo:hi].long()] if row_index is not None else x[lo:hi]
                y[lo:hi] = _expert_mlp_cpu(rows, w_gate_up, w_down, e).to(x.dtype)
        return y
    h = _hip()
    off_ptr = offsets.data_ptr() + 4 * expert0          # the kernels index rows by absolute offsets
    act = torch.empty(rows_bound, dff, dtype=x.dtype, device=dev)
    y = torch.empty(rows_bound, d, dtype=x.dtype, device=dev)
    if zero_unwritten:
        zero_(y)
    # Decode steps (a few dozen routed rows in total): every expert's weights are streamed once
    # against one small panel. Prefill-sized batches use the tiled grouped kernels.
    gg = "lc_gemm_panel_grouped" if rows_bound <= MOE_PANEL_MAX_ROWS else "lc_gemm_grouped"
    if (gg == "lc_gemm_grouped" and rows_bound >= MOE_GEMM256_MIN_ROWS and w_gate_up.n_pad % 256 == 0
            and w_down.n_pad % 256 == 0 and w_gate_up.k % 64 == 0 and w_down.k % 64 == 0):
        # Prefill-sized batches: the 256x256 pipelined tile per expert. It reads contiguous rows,
        # so the rows are first gathered into expert order (a copy of rows_bound rows, a fraction
        # of a percent of the GEMMs' time).
        xs = embed(row_index, x) if row_index is not None else x
        h.call("lc_gemm256_grouped", w_gate_up.data.data_ptr(), w_gate_up.data[0].numel(), xs.data_ptr(), off_ptr,
               E_local, act.data_ptr(), rows_bound, w_gate_up.n, w_gate_up.k, w_gate_up.n_pad, dff, EPI_SWIGLU)
        h.call("lc_gemm256_grouped", w_down.data.data_ptr(), w_down.data[0].numel(), act.data_ptr(), off_ptr,
               E_local, y.data_ptr(), rows_bound, w_down.n, w_down.k, w_down.n_pad, d, EPI_BF16)
        return y
    h.call(gg, w_gate_up.data.data_ptr(), w_gate_up.data[0].numel(), x.data_ptr(), h.ptr(row_index), off_ptr, E_local,
           act.data_ptr(), rows_bound, w_gate_up.n, w_gate_up.k, w_gate_up.n_pad, dff, EPI_SWIGLU)
    h.call(gg, w_down.data.data_ptr(), w_down.data[0].numel(), act.data_ptr(), None, off_ptr, E_local, y.data_ptr(),
           rows_bound, w_down.n, w_down.k, w_down.n_pad, d, EPI_BF16)
    return y


def moe_combine(y: torch.Tensor, slot_of: torch.Tensor, wts: torch.Tensor, T: int,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = sum_k wts[t, k] * y[slot_of[t*k + j]] (fp32 accumulation, activation dtype out;
    written into ``out``, T contiguous rows, when given)."""
    topk = wts.shape[1]
    d = y.shape[1]
    if not y.is_cuda:
        rows = y[slot_of.long()].float().view(T, topk, d)
        res = (rows * wts.float()[:, :, None]).sum(1).to(y.dtype)
        return res if out is None else out.copy_(res)
    h = _hip()
    if out is None:
        out = torch.empty(T, d, dtype=y.dtype, device=y.device)
    h.call("lc_moe_combine", y.data_ptr(), slot_of.data_ptr(), wts.data_ptr(), out.data_ptr(), T, d, topk)
    return out


def moe_experts(x: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, w_gate_up: "ExpertWeights",
                w_down: "ExpertWeights", expert_lo: int = 0, n_experts: Optional[int] = None) -> torch.Tensor:
    """sum_k wts[t,k] * MLP_{ids[t,k]}(x[t]) over the experts held in ``w_*`` (global ids
    [expert_lo, expert_lo + E_local)); (token, k) pairs routed elsewhere contribute zero, so
    expert-parallel ranks can sum their results. ``n_experts`` is the global expert count."""
    T, d = x.shape
    topk = ids.shape[1]
    E_local = w_gate_up.data.shape[0]
    E = n_experts or (expert_lo + E_local)
    offsets, sorted_src, slot_of = moe_permute(ids, E)
    y = experts_on_sorted(x, sorted_src, offsets, expert_lo, w_gate_up, w_down, T * topk, zero_unwritten=E_local != E)
    return moe_combine(y, slot_of, wts, T)


# ---- expert-parallel exchange pieces (parallel/ep.py strings them together) ----
def ep_pack(xs: torch.Tensor, sorted_src: torch.Tensor, offsets: torch.Tensor, slot_of: torch.Tensor, per: int,
            ep: int, cap: int):
    """Send layout of one rank: ``send`` [ep*cap, d] (rows j < count of destination r at
    r*cap + j, in expert-sorted order), ``send_counts`` int32 [ep*per] (pairs per expert) and
    ``slot_back`` int32 [A]: row of the returned [ep*cap, d] buffer holding pair a's output."""
    A = slot_of.numel()
    d = xs.shape[1]
    dev = xs.device
    if not xs.is_cuda:
        send = torch.zeros(ep * cap, d, dtype=xs.dtype)
        off = offsets.long()
        counts = (off[1:] - off[:-1]).to(torch.int32)
        slot_back = torch.empty(A, dtype=torch.int32)
        for r in range(ep):
            lo, hi = int(off[r * per]), int(off[(r + 1) * per])
            send[r * cap: r * cap + hi - lo] = xs[sorted_src[lo:hi].long()]
            m = (slot_of >= lo) & (slot_of < hi)
            slot_back[m] = (r * cap + slot_of[m] - lo).to(torch.int32)
        return send, counts, slot_back
    h = _hip()
    send = torch.empty(ep * cap, d, dtype=xs.dtype, device=dev)
    counts = torch.empty(ep * per, dtype=torch.int32, device=dev)
    slot_back = torch.empty(A, dtype=torch.int32, device=dev)
    h.call("lc_ep_pack", xs.data_ptr(), sorted_src.data_ptr(), offsets.data_ptr(), slot_of.data_ptr(), per, ep, cap, A,
           d, send.data_ptr(), counts.data_ptr(), slot_back.data_ptr())
    return send, counts, slot_back


def ep_recv_index(recv_counts: torch.Tensor, ep: int, per: int, cap: int):
    """From the received per-(source, expert) counts: (row_index int32 [ep*cap]: receive-buffer
    row of every expert-sorted position, offsets_local int32 [per+1])."""
    dev = recv_counts.device
    if not recv_counts.is_cuda:
        c = recv_counts.view(ep, per).long()
        row_index = torch.zeros(ep * cap, dtype=torch.int32)
        offsets = torch.zeros(per + 1, dtype=torch.int32)
        pos = 0
        for e in range(per):
            offsets[e] = pos
            for s in range(ep):
                n, start = int(c[s, e]), int(c[s, :e].sum())
                row_index[pos:pos + n] = torch.arange(s * cap + start, s * cap + start + n, dtype=torch.int32)
                pos += n
        offsets[per] = pos
        return row_index, offsets
    h = _hip()
    row_index = torch.empty(ep * cap, dtype=torch.int32, device=dev)
    offsets = torch.empty(per + 1, dtype=torch.int32, device=dev)
    h.call("lc_ep_recv_index", recv_counts.data_ptr(), ep, per, cap, row_index.data_ptr(), offsets.data_ptr())
    return row_index, offsets


def scatter_rows(y: torch.Tensor, row_index: torch.Tensor, total: torch.Tensor) -> torch.Tensor:
    """out[row_index[p]] = y[p] for p < total[0] (a device integer); other rows are unspecified."""
    if not y.is_cuda:
        out = torch.zeros_like(y)
        n = int(total[0])
        out[row_index[:n].long()] = y[:n]
        return out
    h = _hip()
    out = torch.empty_like(y)
    h.call("lc_scatter_rows", y.data_ptr(), row_index.data_ptr(), total.data_ptr(), y.shape[0], y.shape[1], out.data_ptr())
    return out


def moe_ffn(x: torch.Tensor, Wr: torch.Tensor, w_gate_up: ExpertWeights, w_down: ExpertWeights, topk: int,
            expert_lo: int = 0) -> torch.Tensor:
    """Mixtral block-sparse FFN: route, run the selected experts' SwiGLU MLP, combine. With a
    subset of the experts resident (``expert_lo``, stacked weights shorter than the router)
    the result is this rank's partial sum."""
    ids, wts = moe_route(x, Wr, topk)
    return moe_experts(x, ids, wts, w_gate_up, w_down, expert_lo, Wr.shape[0])


# ---------------------------------------------------------------------------- hybrid decoders
# Ops of hybrid decoder designs (csrc/kernels/hybrid.hip): an fp32 residual stream with scalar-gain
# norms on the sublayer outputs, recurrences over per-sequence state slots, attention with separate
# key / value widths under a chunk or window mask. ``act_dtype`` (bf16 or fp32) is the type of what
# feeds the next matrix product; everything else is fp32. CPU tensors go to ops.reference.
def _f32flag(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return 1
    if dtype == torch.bfloat16:
        return 0
    raise TypeError(f"activation type {dtype}: bf16 or fp32")


def linear_any(x: torch.Tensor, w: LinearWeight, out_f32: bool = True, epi_relu2: bool = False) -> torch.Tensor:
    """y = x W^T (+ bias) for a row-major weight of any shape and type (fp32 accumulation on the
    vector ALUs). ``epi_relu2``: the square of relu in the epilogue."""
    M = x.shape[0]
    odt = torch.float32 if out_f32 else torch.bfloat16
    if x.shape[1] != w.k:
        raise ValueError(f"linear_any: activations of width {x.shape[1]} against a weight of depth {w.k}")
    if not x.is_cuda:
        y = ref.linear(x, w.dense(), w.bias, torch.float32)
        return (torch.relu(y).pow(2) if epi_relu2 else y).to(odt)
    if w.is_packed:
        raise ValueError("linear_any takes row-major weights")
    if x.stride(1) != 1:
        x = x.contiguous()              # (a column slice of a wider matrix is taken as it is)
    y = torch.empty(M, w.n, dtype=odt, device=x.device)
    _hip().call("lc_gemm_any", x.data_ptr(), _f32flag(x.dtype), x.stride(0) if M > 1 else max(x.stride(0), w.k),
                w.data.data_ptr(), _f32flag(w.data.dtype),
                _hip().ptr(w.bias), y.data_ptr(), 1 if out_f32 else 0, M, w.n, w.k, 1 if epi_relu2 else 0)
    return y


def embed_rows(ids: torch.Tensor, E: torch.Tensor, act_dtype: Optional[torch.dtype],
               feed: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, scale: float = 1.0,
               positions: Optional[torch.Tensor] = None, inv_freq: Optional[torch.Tensor] = None):
    """Rows E[ids] * scale as (fp32 [T, d], copy in ``act_dtype`` or None). E is bf16 or fp32; with
    ``act_dtype`` fp32 the copy IS the fp32 tensor. ``feed`` as in ``embed``. With ``positions`` and
    ``inv_freq`` (fp64 [d/2]) a sinusoidal position vector is added: entry 2i is sin(p f_i), entry
    2i + 1 cos(p f_i), the angle and its reduction in fp64. Also the row gather of an fp32 matrix."""
    T, d = ids.numel(), E.shape[1]
    if inv_freq is not None and (positions is None or 2 * inv_freq.numel() != d or inv_freq.dtype != torch.float64):
        raise ValueError("embed_rows: the position table needs positions and d / 2 fp64 frequencies")
    if not ids.is_cuda:
        if feed is not None:
            tok, rows = feed
            ids = torch.where(rows >= 0, tok[rows.clamp_min(0).long()].to(ids.dtype), ids)
        x = ref.embed(ids, E).float()
        if scale != 1.0:
            x = x * scale
        if inv_freq is not None:
            x = x + ref.sinusoid_rows(positions, inv_freq)
        return x, (x if act_dtype in (None, torch.float32) else x.to(act_dtype))
    x = torch.empty(T, d, dtype=torch.float32, device=E.device)
    xa = torch.empty(T, d, dtype=act_dtype, device=E.device) if act_dtype == torch.bfloat16 else None
    _hip().call("lc_embed_rows", ids.data_ptr(), E.data_ptr(), _f32flag(E.dtype), x.data_ptr(), _hip().ptr(xa), 0, T, d,
                E.shape[0], feed[0].data_ptr() if feed is not None else None,
                feed[1].data_ptr() if feed is not None else None, float(scale),
                positions.data_ptr() if inv_freq is not None else None, _hip().ptr(inv_freq))
    return x, (xa if xa is not None else (x if act_dtype is not None else None))


def scalar_norm_add(x: torch.Tensor, y: Optional[torch.Tensor], gain: torch.Tensor, eps: float,
                    act_dtype: torch.dtype) -> torch.Tensor:
    """x (fp32 residual stream, in place) += y / sqrt(mean(y^2) + eps) * gain and the new x in
    ``act_dtype``; without ``y``: the normed x in ``act_dtype`` (x untouched). ``gain`` is an
    fp32 tensor of one element."""
    if not x.is_cuda:
        return ref.scalar_norm_add(x, y, gain, eps, act_dtype)
    T, d = x.shape
    if y is not None and (y.shape != x.shape or y.dtype != torch.float32):
        raise ValueError("scalar_norm_add: the sublayer output must be fp32 of the stream's shape")
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError("scalar_norm_add: the residual stream is a contiguous fp32 tensor")
    alias = y is not None and act_dtype == torch.float32       # the fp32 'copy' is the stream itself
    xa = None if alias else torch.empty(T, d, dtype=act_dtype, device=x.device)
    _hip().call("lc_scalar_norm_add", x.data_ptr(), _hip().ptr(y.contiguous() if y is not None else None),
                gain.data_ptr(), float(eps), _hip().ptr(xa), _f32flag(act_dtype), T, d)
    return x if alias else xa


def relu2(y: torch.Tensor, act_dtype: torch.dtype) -> torch.Tensor:
    """relu(y)^2 of an fp32 matrix (may be a column slice of a wider one) in ``act_dtype``."""
    if not y.is_cuda:
        return ref.relu2(y, act_dtype)
    if y.dim() != 2 or y.stride(1) != 1 or y.dtype != torch.float32:
        raise ValueError("relu2: an fp32 matrix with unit column stride")
    T, cols = y.shape
    out = torch.empty(T, cols, dtype=act_dtype, device=y.device)
    _hip().call("lc_relu2", y.data_ptr(), out.data_ptr(), _f32flag(act_dtype), T, cols, max(y.stride(0), cols))
    return out


def _scan_scratch(B: int, max_len: int, state_floats: int, decay_floats: int, device) -> Optional[torch.Tensor]:
    """Carry buffer of the segmented scans (portions longer than two segments of 32 rows run as
    segments side by side: hybrid.hip), None when the step's portions are short."""
    n = int(_hip().lib().lc_scan_scratch_floats(B, int(max_len), state_floats, decay_floats))
    return torch.empty(n, dtype=torch.float32, device=device) if n else None


def mingru_scan(zxg: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor,
                slots: torch.Tensor, act_dtype: torch.dtype, max_len: int = 1) -> torch.Tensor:
    """minGRU over the step's sequences: zxg fp32 [T, 3w] (update-gate logits | candidate
    pre-activations | output-gate logits), state fp32 [slots, w] (updated in place). Returns
    S * silu(g) [T, w] in ``act_dtype``. ``max_len``: the longest portion of the step (host-known;
    long portions are scanned in parallel segments)."""
    if not zxg.is_cuda:
        return ref.mingru_scan(zxg, state, cu_q, positions, slots, act_dtype)
    T, w = zxg.shape[0], zxg.shape[1] // 3
    if zxg.dtype != torch.float32 or state.dtype != torch.float32 or state.shape[1] != w:
        raise ValueError("mingru_scan: fp32 projections [T, 3w] and fp32 state [slots, w]")
    zxg = zxg.contiguous()
    out = torch.empty(T, w, dtype=act_dtype, device=zxg.device)
    B = slots.numel()
    scratch = _scan_scratch(B, max_len, w, w, zxg.device)
    _hip().call("lc_mingru_scan", zxg.data_ptr(), state.data_ptr(), cu_q.data_ptr(), positions.data_ptr(),
                slots.data_ptr(), out.data_ptr(), _f32flag(act_dtype), B, w, int(max_len), _hip().ptr(scratch))
    return out


def gla_scan(proj: torch.Tensor, decay_logits: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor,
             positions: torch.Tensor, slots: torch.Tensor, H: int, D: int, Dv: int, tau: float,
             max_len: int = 1) -> torch.Tensor:
    """Gated linear attention over the step's sequences. proj fp32 [T, >= 2HD + HDv] holds
    q | k | v in its first columns, decay_logits fp32 [T, HD]; state fp32 [slots, H*D*Dv]
    (updated in place). Returns the un-normed read-out fp32 [T, H*Dv]. ``max_len`` as in
    ``mingru_scan``."""
    if not proj.is_cuda:
        return ref.gla_scan(proj, decay_logits, state, cu_q, positions, slots, H, D, Dv, tau)
    T = proj.shape[0]
    if proj.dtype != torch.float32 or decay_logits.dtype != torch.float32 or state.dtype != torch.float32:
        raise ValueError("gla_scan: fp32 inputs and state")
    if state.shape[1] != H * D * Dv or decay_logits.shape[1] != H * D or proj.stride(1) != 1:
        raise ValueError("gla_scan: shapes do not fit the head sizes")
    decay_logits = decay_logits.contiguous()
    out = torch.empty(T, H * Dv, dtype=torch.float32, device=proj.device)
    B = slots.numel()
    scratch = _scan_scratch(B, max_len, H * D * Dv, H * D, proj.device)
    prep = torch.empty(T * H * D * 4, dtype=torch.float32, device=proj.device)     # (q, k, decay, -) per channel
    _hip().call("lc_gla_scan", proj.data_ptr(), proj.stride(0), decay_logits.data_ptr(), state.data_ptr(),
                state.stride(0), cu_q.data_ptr(), positions.data_ptr(), slots.data_ptr(), out.data_ptr(), T, B, H, D, Dv,
                float(tau), int(max_len), _hip().ptr(scratch), prep.data_ptr())
    return out


def headnorm_gate(o: torch.Tensor, w: torch.Tensor, gate: torch.Tensor, Dv: int, eps: float,
                  act_dtype: torch.dtype) -> torch.Tensor:
    """Per head of width Dv: o / sqrt(mean(o^2) + eps) * w, times silu(gate). ``gate`` may be a
    column slice of a wider fp32 matrix."""
    if not o.is_cuda:
        return ref.headnorm_gate(o, w, gate, Dv, eps, act_dtype)
    T, n = o.shape
    if gate.shape != o.shape or gate.stride(1) != 1 or o.dtype != torch.float32 or gate.dtype != torch.float32:
        raise ValueError("headnorm_gate: fp32 read-out and gate of one shape")
    o = o.contiguous()
    out = torch.empty(T, n, dtype=act_dtype, device=o.device)
    _hip().call("lc_headnorm_gate", o.data_ptr(), w.data_ptr(), gate.data_ptr(), gate.stride(0), out.data_ptr(),
                _f32flag(act_dtype), T, n // Dv, Dv, float(eps), Dv, 0, 0, None)
    return out


def qkv_prep(qkv: torch.Tensor, q_norm: torch.Tensor, k_norm: Optional[torch.Tensor], inv_freq: torch.Tensor,
             positions: torch.Tensor, slot_mapping: torch.Tensor, k_cache: Optional[torch.Tensor],
             v_cache: Optional[torch.Tensor], H: int, G: int, D: int, Dv: int, rot_dims: int, rot_base: float,
             eps: float) -> torch.Tensor:
    """Attention pre-processing in one launch: RMS norm of the whole query (and key) projection
    with per-coordinate weights, partial rotate-half rotary positions, unit-RMS value heads, and
    the write of keys [blocks, G, BS, D] / values [blocks, G, BS, Dv] at the rows' slots. A layer
    that reads another layer's keys passes no caches. Returns q fp32 [T, H*D]."""
    if not qkv.is_cuda:
        return ref.qkv_prep(qkv, q_norm, k_norm, positions, slot_mapping, k_cache, v_cache, H, G, D, Dv, rot_dims,
                            rot_base, eps)
    T = qkv.shape[0]
    if qkv.dtype != torch.float32 or qkv.stride(1) != 1:
        raise ValueError("qkv_prep: fp32 projections")
    has_kv = k_cache is not None
    if has_kv and (k_cache.dtype != v_cache.dtype or k_cache.shape[1:] != (G, k_cache.shape[2], D)
                   or v_cache.shape[1:] != (G, k_cache.shape[2], Dv)):
        raise ValueError("qkv_prep: cache planes do not fit the head sizes")
    q = torch.empty(T, H * D, dtype=torch.float32, device=qkv.device)
    _hip().call("lc_qkv_prep", qkv.data_ptr(), qkv.stride(0), q_norm.data_ptr(), _hip().ptr(k_norm), inv_freq.data_ptr(),
                positions.data_ptr(), slot_mapping.data_ptr(), _hip().ptr(k_cache), _hip().ptr(v_cache),
                _f32flag(k_cache.dtype) if has_kv else 0, q.data_ptr(), T, H, G, D, Dv,
                k_cache.shape[2] if has_kv else 1, rot_dims, float(eps), 1 if has_kv else 0)
    return q


def attn_tile_ok(D: int, Dv: int) -> bool:
    """Whether prompt portions of these head widths take the matrix-core kernel (fp32 MFMA tiles:
    widths in whole MFMA steps, up to 256 value columns, one block's tiles within 160 KB of LDS);
    otherwise the row kernel."""
    if D % 8 or Dv % 16 or Dv > 256 or D > 256:
        return False
    ds, vs = D + ((4 - D % 32 + 32) % 32), Dv + ((16 - Dv % 32 + 32) % 32)
    return (80 * ds + 16 * vs + 4 * 16 * 17) * 4 <= 160 * 1024


ATTN_TILE_MIN_ROWS = int(os.environ.get("LC_ATTN_TILE_MIN_ROWS", "16"))


def _cache_ld(c: torch.Tensor, G: int, width: int, what: str) -> int:
    """Row stride of a cache plane [blocks, G, BS, width] that may be a column block of wider rows."""
    BS, ld = c.shape[2], c.stride(2)
    if c.dim() != 4 or c.shape[1] != G or c.shape[3] != width or c.stride(3) != 1 or ld < width or \
            c.stride(1) != BS * ld or c.stride(0) != G * BS * ld:
        raise ValueError(f"attn_masked: the {what} plane does not fit the head sizes")
    return ld


def attn_masked(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                cu_q: torch.Tensor, row_seq: torch.Tensor, positions: torch.Tensor, H: int, G: int, D: int, Dv: int,
                scale: float, chunk: int, window: int, act_dtype: torch.dtype, n_portions: int = 0,
                portion_rows: int = 0, max_len: int = 0, softcap: float = 0.0, sink: bool = False,
                all_value_heads: bool = False) -> torch.Tensor:
    """Attention of fp32 queries [T, H*D] over paged keys / values of widths D / Dv. The row at
    position p sees keys j <= p with j >= floor(p / chunk) * chunk (``chunk`` > 0) and
    j > p - window (``window`` > 0), counted from the start of its sequence. ``row_seq`` [T]
    names each row's sequence (row of ``block_tables``); scores, weights and sums are fp32.
    The planes are [blocks, G, BS, D] / [blocks, G, BS, Dv] and may be column blocks of wider rows
    (a latent row that is key and value at once). ``softcap`` > 0: the scaled score s becomes
    softcap * tanh(s / softcap). ``sink``: the softmax has a silent extra entry of score 0, so the
    weights sum to less than one. ``all_value_heads``: every query head's weights are applied to
    the values of ALL G key/value heads; the result is [T, H * G * Dv] (head, value head, column).

    Two kernels: the first ``n_portions`` sequences (rows [0, portion_rows), the longest of
    ``max_len`` rows) are prompt portions and go, 64 rows of a head per block, through fp32 MFMA
    tiles; the rows behind them (single decoded tokens) and shapes the tiles do not take go
    through the row kernel, one wave per (row, head)."""
    if not q.is_cuda:
        return ref.attn_masked(q, k_cache, v_cache, block_tables, cu_q, positions, H, G, D, Dv, scale, chunk, window,
                               act_dtype, softcap, sink, all_value_heads)
    T = q.shape[0]
    if q.dtype != torch.float32 or not q.is_contiguous() or k_cache.dtype != v_cache.dtype:
        raise ValueError("attn_masked: contiguous fp32 queries, caches of one type")
    k_ld, v_ld = _cache_ld(k_cache, G, D, "key"), _cache_ld(v_cache, G, Dv, "value")
    if k_cache.shape[2] != v_cache.shape[2]:
        raise ValueError("attn_masked: key and value planes of one block size")
    if not 0 <= portion_rows <= T or n_portions > block_tables.shape[0]:
        raise ValueError("attn_masked: the portions exceed the step")
    nv = G if all_value_heads else 1
    o_ld = nv * Dv
    out = torch.empty(T, H * o_ld, dtype=act_dtype, device=q.device)
    BS, MB, cf, af = k_cache.shape[2], block_tables.shape[1], _f32flag(k_cache.dtype), _f32flag(act_dtype)

    def value_groups(cap: int):
        """(first value head or -1, heads, first output column) per launch: as many value heads side by side as fit."""
        if not all_value_heads:
            return [(-1, 1, 0)] if Dv <= cap else []
        n = cap // Dv
        return [(v0, min(n, G - v0), v0 * Dv) for v0 in range(0, G, n)] if n else []
    opts = (float(softcap), 1 if sink else 0)
    first = 0
    # value heads side by side in one tile: equal groups whose width the tiles take (whole MFMA steps of 16 columns)
    tile_cols = max([n * Dv for n in range(1, nv + 1) if nv % n == 0 and Dv % 8 == 0 and attn_tile_ok(D, n * Dv)] or [0])
    aligned = k_ld % 8 == 0 and v_ld % 8 == 0 and k_cache.data_ptr() % 16 == 0 and v_cache.data_ptr() % 16 == 0
    if n_portions > 0 and portion_rows > 0 and max_len >= ATTN_TILE_MIN_ROWS and tile_cols and aligned:
        for vh0, nvh, col0 in value_groups(tile_cols):
            _hip().call("lc_attn_tile", q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), cf, block_tables.data_ptr(),
                        MB, cu_q.data_ptr(), positions.data_ptr(), out.data_ptr(), af, int(n_portions), int(max_len), H, G,
                        D, Dv, BS, float(scale), int(chunk), int(window), k_ld, v_ld, *opts, vh0, nvh, o_ld, col0)
        first = portion_rows
    if first < T:
        if Dv > 512:
            raise ValueError("attn_masked: the row kernel takes value widths up to 512")
        # (value heads side by side: a block along z per value head; the short rows' scores are formed again there)
        _hip().call("lc_attn_masked", q[first:].data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), cf,
                    block_tables.data_ptr(), MB, row_seq[first:].data_ptr(), positions[first:].data_ptr(),
                    out[first:].data_ptr(), af, T - first, H, G, D, Dv, BS, float(scale), int(chunk), int(window),
                    k_ld, v_ld, *opts, 0 if all_value_heads else -1, 1, o_ld, 0, nv)
    return out


# ---- pre-norm designs, latent attention, mLSTM, routed feed-forwards (hybrid.hip, hybrid_moe.hip) ----
def add_rmsnorm(x: torch.Tensor, y: Optional[torch.Tensor], w: Optional[torch.Tensor], eps: float,
                act_dtype: torch.dtype) -> Optional[torch.Tensor]:
    """The residual step of a pre-norm layer in one launch: x (fp32 stream, in place) += y, and the
    input of the next sublayer x / sqrt(mean(x^2) + eps) * w in ``act_dtype`` (``w``: fp32 [d], any
    offset already folded in). Without ``y`` only the norm; without ``w`` only the sum (returns None)."""
    if not x.is_cuda:
        return ref.add_rmsnorm(x, y, w, eps, act_dtype)
    T, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError("add_rmsnorm: the residual stream is a contiguous fp32 tensor")
    if y is not None and (y.shape != x.shape or y.dtype != torch.float32):
        raise ValueError("add_rmsnorm: the sublayer output must be fp32 of the stream's shape")
    if y is None and w is None:
        return None
    xa = torch.empty(T, d, dtype=act_dtype, device=x.device) if w is not None else None
    _hip().call("lc_add_rmsnorm", x.data_ptr(), _hip().ptr(y.contiguous() if y is not None else None), _hip().ptr(w),
                float(eps), _hip().ptr(xa), _f32flag(act_dtype), T, d)
    return xa


def latent_write(proj: torch.Tensor, col0: int, w: torch.Tensor, eps: float, slot_mapping: torch.Tensor,
                 cache: torch.Tensor) -> None:
    """The compressed key/value row of every token: rms_norm(proj[:, col0:col0 + R]) * w, written to
    ``cache`` [blocks, 1, BS, R] at the rows' slots (rows with slot < 0 are skipped)."""
    if not proj.is_cuda:
        return ref.latent_write(proj, col0, w, eps, slot_mapping, cache)
    R = cache.shape[3]
    if proj.dtype != torch.float32 or proj.stride(1) != 1 or cache.shape[1] != 1 or col0 + R > proj.shape[1]:
        raise ValueError("latent_write: fp32 projections and a one-head cache plane of the latent's width")
    _hip().call("lc_latent_write", proj.data_ptr(), proj.stride(0), int(col0), R, w.data_ptr(), float(eps),
                slot_mapping.data_ptr(), cache.data_ptr(), _f32flag(cache.dtype), cache.shape[2], proj.shape[0])


def head_linear(x: torch.Tensor, W: torch.Tensor, out_dtype: torch.dtype, gate: Optional[torch.Tensor] = None,
                x_head_stride: Optional[int] = None, out: Optional[torch.Tensor] = None,
                out_head_stride: Optional[int] = None, gate_full: bool = False) -> torch.Tensor:
    """Per-head products y[t, h] = W[h] x[t, h]: x [T, >= H*K] (may be a column slice), W [H, N, K]
    row-major, y [T, H*N] in ``out_dtype``; fp32 accumulation. ``gate`` [T, H] (logits, may be a
    column slice): y[t, h] *= sigmoid(gate[t, h]); with ``gate_full`` the gate is [T, H*N], a logit per
    output. ``x_head_stride``: head h's inputs start at column h * x_head_stride (default K: heads side by
    side). ``out`` / ``out_head_stride``: write head h's outputs from column h * out_head_stride of this
    matrix instead of a new one (the other columns are left alone)."""
    H, N, K = W.shape
    M = x.shape[0]
    xs = K if x_head_stride is None else int(x_head_stride)
    os_ = N if out_head_stride is None else int(out_head_stride)
    if xs < K or x.shape[1] < (H - 1) * xs + K or x.stride(1) != 1 or not W.is_contiguous():
        raise ValueError("head_linear: activations [T, H*K] against weights [H, N, K]")
    if gate is not None and (gate.shape != (M, H * N if gate_full else H) or gate.dtype != torch.float32 or gate.stride(1) != 1):
        raise ValueError("head_linear: the gate is an fp32 [T, H] matrix ([T, H*N] when it is a logit per output)")
    if gate is None and gate_full:
        raise ValueError("head_linear: a gate per output needs the gate")
    if out is not None and (out.shape[0] != M or out.dtype != out_dtype or out.stride(1) != 1 or os_ < N
                            or out.shape[1] < (H - 1) * os_ + N):
        raise ValueError("head_linear: the output matrix does not hold the heads' blocks")
    if not x.is_cuda:
        return ref.head_linear(x, W, out_dtype, gate, xs, out, os_, gate_full)
    y = out if out is not None else torch.empty(M, (H - 1) * os_ + N, dtype=out_dtype, device=x.device)
    _hip().call("lc_head_linear", x.data_ptr(), _f32flag(x.dtype), max(x.stride(0), (H - 1) * xs + K), W.data_ptr(),
                _f32flag(W.dtype), y.data_ptr(), _f32flag(out_dtype), _hip().ptr(gate),
                max(gate.stride(0), gate.shape[1]) if gate is not None else 0, M, H, N, K, xs,
                max(y.stride(0), (H - 1) * os_ + N), os_, 1 if gate_full else 0)
    return y


def mlstm_scan(proj: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor,
               slots: torch.Tensor, H: int, D: int, Dv: int, cap: float, max_len: int = 1):
    """mLSTM matrix memory over the step's sequences. proj fp32 [T, >= 2HD + 2HDv + 2H] holds
    q | k | v | output gate | input-gate logits | forget-gate logits; state fp32
    [slots, H*D*(Dv+1) + H] (per head S with the normaliser as an extra column, then the running
    maxima; updated in place). Gates are soft-capped (``cap`` > 0). Returns (read-out fp32
    [T, H*(Dv+1)], last column per head = normaliser . q; running maximum fp32 [T, H])."""
    if not proj.is_cuda:
        return ref.mlstm_scan(proj, state, cu_q, positions, slots, H, D, Dv, cap)
    T = proj.shape[0]
    need = 2 * H * D + 2 * H * Dv + 2 * H
    if proj.dtype != torch.float32 or state.dtype != torch.float32 or proj.stride(1) != 1 or proj.shape[1] < need:
        raise ValueError("mlstm_scan: fp32 projections q | k | v | g | i | f and fp32 state")
    if state.shape[1] != H * D * (Dv + 1) + H or D > 256:
        raise ValueError("mlstm_scan: the state does not fit the head sizes (key width at most 256)")
    B = slots.numel()
    Da = Dv + 1
    out = torch.empty(T, H * Da, dtype=torch.float32, device=proj.device)
    m = torch.empty(T, H, dtype=torch.float32, device=proj.device)
    prep = torch.empty(T * H * (4 * D + 2), dtype=torch.float32, device=proj.device)    # operands, then (a, b) per (token, head)
    scratch = _scan_scratch(B, max_len, H * D * Da, H * D, proj.device)
    _hip().call("lc_mlstm_scan", proj.data_ptr(), proj.stride(0), state.data_ptr(), state.stride(0), cu_q.data_ptr(),
                positions.data_ptr(), slots.data_ptr(), out.data_ptr(), m.data_ptr(), T, B, H, D, Dv, float(cap),
                int(max_len), _hip().ptr(scratch), prep.data_ptr())
    return out, m


def mlstm_out(o: torch.Tensor, m: torch.Tensor, w: torch.Tensor, gate: torch.Tensor, H: int, Dv: int, eps: float,
              act_dtype: torch.dtype) -> torch.Tensor:
    """From ``mlstm_scan``'s read-out: per head o[:Dv] / (max(|o[Dv]|, exp(-m)) + 1e-6), scaled to
    unit RMS, times w [H*Dv], times sigmoid(gate) (fp32 [T, H*Dv], may be a column slice)."""
    if not o.is_cuda:
        return ref.mlstm_out(o, m, w, gate, H, Dv, eps, act_dtype)
    T = o.shape[0]
    if o.shape[1] != H * (Dv + 1) or gate.shape != (T, H * Dv) or gate.stride(1) != 1 or w.numel() != H * Dv:
        raise ValueError("mlstm_out: shapes do not fit the head sizes")
    out = torch.empty(T, H * Dv, dtype=act_dtype, device=o.device)
    _hip().call("lc_headnorm_gate", o.data_ptr(), w.data_ptr(), gate.data_ptr(), gate.stride(0), out.data_ptr(),
                _f32flag(act_dtype), T, H, Dv, float(eps), Dv + 1, Dv, 1, m.data_ptr())
    return out


def glu(y: torch.Tensor, act_dtype: torch.dtype, kind: str = "relu") -> torch.Tensor:
    """fp32 y [T, 2n] = (gate | up) -> act(gate) * up [T, n] in ``act_dtype`` (act: relu or silu)."""
    if not y.is_cuda:
        return ref.glu(y, act_dtype, kind)
    T, n = y.shape[0], y.shape[1] // 2
    y = y.contiguous()
    out = torch.empty(T, n, dtype=act_dtype, device=y.device)
    _hip().call("lc_glu", y.data_ptr(), out.data_ptr(), _f32flag(act_dtype), T, n, {"relu": 0, "silu": 1}[kind])
    return out


def route_grouped(z: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int, keep: int, scale: float,
                  score: str = "softmax"):
    """Group-limited top-k routing over fp32 router logits z [T, n] (see ops.reference.route_grouped):
    (ids int32 [T, top], weights fp32 [T, top]). ``score``: softmax over the outputs, or sigmoid of each;
    ``correction`` may be None."""
    if score not in ("softmax", "sigmoid"):
        raise ValueError(f"route_grouped: score function {score!r}: softmax or sigmoid")
    T, n = z.shape
    if groups < 1 or n % groups or not 1 <= keep <= groups or top > keep * (n // groups):
        raise ValueError("route_grouped: groups must divide the router's width and the kept groups hold `top` outputs")
    if not z.is_cuda:
        return ref.route_grouped(z, correction, top, groups, keep, scale, score)
    if z.stride(1) != 1 or z.dtype != torch.float32:
        raise ValueError("route_grouped: fp32 logits (a column slice of a wider matrix is taken as it is)")
    ids = torch.empty(T, top, dtype=torch.int32, device=z.device)
    wts = torch.empty(T, top, dtype=torch.float32, device=z.device)
    _hip().call("lc_route_grouped", z.data_ptr(), max(z.stride(0), n), _hip().ptr(correction), T, n, top, groups, keep,
                float(scale), 1 if score == "sigmoid" else 0, ids.data_ptr(), wts.data_ptr())
    return ids, wts


def moe_sort(ids: torch.Tensor, n: int, wts: Optional[torch.Tensor] = None):
    """``moe_permute`` for any number of experts (one block, counting sort): (offsets int32 [n+1],
    sorted_src int32 [T*k], slot_of int32 [T*k]); with ``wts`` (fp32 [T, k]) also the weights in sorted
    order, fp32 [T*k], as a fourth result."""
    if not ids.is_cuda:
        offsets, sorted_src, slot_of = moe_permute(ids, n)
        if wts is None:
            return offsets, sorted_src, slot_of
        sw = torch.zeros(ids.numel(), dtype=torch.float32)
        sw[slot_of.long()] = wts.reshape(-1).float()
        return offsets, sorted_src, slot_of, sw
    T, topk = ids.shape
    dev = ids.device
    offsets = torch.empty(n + 1, dtype=torch.int32, device=dev)
    sorted_src = torch.empty(T * topk, dtype=torch.int32, device=dev)
    slot_of = torch.empty(T * topk, dtype=torch.int32, device=dev)
    sw = torch.empty(T * topk, dtype=torch.float32, device=dev) if wts is not None else None
    if wts is not None and (wts.dtype != torch.float32 or wts.numel() != ids.numel() or not wts.is_contiguous()):
        raise ValueError("moe_sort: fp32 weights, one per (token, choice) pair")
    _hip().call("lc_moe_sort", ids.data_ptr(), T, topk, n, offsets.data_ptr(), sorted_src.data_ptr(), slot_of.data_ptr(),
                _hip().ptr(wts), _hip().ptr(sw))
    return (offsets, sorted_src, slot_of) if wts is None else (offsets, sorted_src, slot_of, sw)


def grouped_linear(x: torch.Tensor, row_index: Optional[torch.Tensor], offsets: torch.Tensor, W,
                   out_dtype: torch.dtype, rows: int, relu2_epi: bool = False, glu_clamp=None) -> torch.Tensor:
    """Per-expert products over expert-sorted rows: position p in [offsets[e], offsets[e+1]) gives
    W[e] x[row_index[p]] (x[p] without an index); ``relu2_epi``: square of relu. W is either a
    row-major tensor [E, N, K] of any shape and type (fp32 accumulation on the vector ALUs) or
    packed ``ExpertWeights`` (bf16 activations, the grouped MFMA kernels: one panel per expert for a
    few hundred rows, 128 x 128 tiles beyond). Positions of experts >= E are left unwritten.
    ``glu_clamp`` = (row_scale fp32 [rows] or None, limit, slope, shift), packed weights marked ``swiglu``
    only (16-row tiles alternate gate / up, ``interleave_gate_up``): the clamped gated unit of the product,
    scaled per sorted row, as the epilogue; the result is bf16 [rows, N / 2]."""
    if glu_clamp is not None:
        if not (isinstance(W, ExpertWeights) and W.swiglu and x.is_cuda and W.n % 32 == 0):
            raise ValueError("grouped_linear: the gated epilogue takes packed gate / up tiles on the GPU")
        if x.dtype != torch.bfloat16 or x.shape[1] != W.k or not x.is_contiguous() or out_dtype != torch.bfloat16:
            raise ValueError("grouped_linear: packed experts take contiguous bf16 activations of their depth")
        scale, limit, slope, shift = glu_clamp
        if scale is not None and (scale.dtype != torch.float32 or scale.numel() < rows):
            raise ValueError("grouped_linear: one fp32 scale per sorted row")
        y = torch.empty(rows, W.n // 2, dtype=torch.bfloat16, device=x.device)
        gg = "lc_gemm_panel_grouped_glu" if rows <= MOE_PANEL_MAX_ROWS else "lc_gemm_grouped_glu"
        _hip().call(gg, W.data.data_ptr(), W.data[0].numel(), x.data_ptr(), _hip().ptr(row_index), offsets.data_ptr(),
                    W.data.shape[0], y.data_ptr(), int(rows), W.n, W.k, W.n_pad, W.n // 2, _hip().ptr(scale), float(limit),
                    float(slope), float(shift))
        return y
    if isinstance(W, ExpertWeights) and W.swiglu:
        raise ValueError("grouped_linear: interleaved gate / up tiles need the gated epilogue")
    if isinstance(W, ExpertWeights) and W.data.dim() == 3:
        W = W.data                                    # CPU: [E, N, K]
    if not x.is_cuda:
        return ref.grouped_linear(x, row_index, offsets, W, out_dtype, rows, relu2_epi)
    if isinstance(W, ExpertWeights):
        if x.dtype != torch.bfloat16 or x.shape[1] != W.k or not x.is_contiguous():
            raise ValueError("grouped_linear: packed experts take contiguous bf16 activations of their depth")
        if relu2_epi and out_dtype != torch.bfloat16:
            raise ValueError("grouped_linear: the relu^2 epilogue of the packed kernels writes bf16")
        y = torch.empty(rows, W.n, dtype=out_dtype, device=x.device)
        epi = 3 if relu2_epi else (EPI_F32 if out_dtype == torch.float32 else EPI_BF16)
        gg = "lc_gemm_panel_grouped" if rows <= MOE_PANEL_MAX_ROWS else "lc_gemm_grouped"
        _hip().call(gg, W.data.data_ptr(), W.data[0].numel(), x.data_ptr(), _hip().ptr(row_index), offsets.data_ptr(),
                    W.data.shape[0], y.data_ptr(), int(rows), W.n, W.k, W.n_pad, W.n, epi)
        return y
    E, N, K = W.shape
    if x.shape[1] != K or x.stride(1) != 1 or not W.is_contiguous():
        raise ValueError("grouped_linear: activations of the experts' depth")
    y = torch.empty(rows, N, dtype=out_dtype, device=x.device)
    _hip().call("lc_gemm_any_grouped", x.data_ptr(), _f32flag(x.dtype), max(x.stride(0), K), _hip().ptr(row_index),
                offsets.data_ptr(), W.data_ptr(), _f32flag(W.dtype), y.data_ptr(), _f32flag(out_dtype), int(rows), E, N, K,
                1 if relu2_epi else 0)
    return y


def moe_mix(ye: torch.Tensor, slot_of: torch.Tensor, ids: torch.Tensor, wts: Optional[torch.Tensor], h: torch.Tensor, E: int,
            shared: Optional[torch.Tensor] = None, shared_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 [T, d] = sum_k wts[t, k] * (ye[slot_of[t, k]] if ids[t, k] < E else h[t]) (+ shared[t]):
    experts with ids >= E are identity experts, whose output is the feed-forward's input itself.
    Without ``wts`` every chosen expert counts once. ``shared_gate`` (fp32 logits [T, 1], may be a column
    of a wider matrix): the shared expert's row is scaled by sigmoid(shared_gate[t])."""
    if not ye.is_cuda:
        return ref.moe_mix(ye, slot_of, ids, wts, h, E, shared, shared_gate)
    if shared_gate is not None and (shared is None or shared_gate.dtype != torch.float32 or shared_gate.shape != (ids.shape[0], 1)):
        raise ValueError("moe_mix: the shared expert's gate is an fp32 [T, 1] column")
    T, top = ids.shape
    d = h.shape[1]
    if ye.dtype != torch.float32 or (shared is not None and shared.dtype != torch.float32):
        raise ValueError("moe_mix: fp32 expert outputs")
    out = torch.empty(T, d, dtype=torch.float32, device=h.device)
    _hip().call("lc_moe_mix", ye.data_ptr(), slot_of.data_ptr(), ids.data_ptr(), _hip().ptr(wts), h.contiguous().data_ptr(),
                _f32flag(h.dtype), _hip().ptr(shared), _hip().ptr(shared_gate),
                max(1, shared_gate.stride(0)) if shared_gate is not None else 0, out.data_ptr(), T, d, top, E)
    return out


# ---- Dynamic Tanh norms, attention whose values are its un-rotated keys, clamped gated experts (hybrid.hip) ----
def add_dyt(x: torch.Tensor, y: Optional[torch.Tensor], mult: float, alpha: float, w: Optional[torch.Tensor],
            b: Optional[torch.Tensor], act_dtype: Optional[torch.dtype], out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """The residual step of a layer whose norm is a Dynamic Tanh, one launch: x (fp32 stream, in place)
    += mult * y, and tanh(alpha * x) * w + b in ``act_dtype`` (w, b: fp32 [d]). Without ``y`` only the norm;
    without ``w`` the stream itself in the activation type (or nothing, when ``act_dtype`` is None too).
    ``out``: where the result goes, a [T, d] column block of a wider matrix (default: a new tensor)."""
    T, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError("add_dyt: the residual stream is a contiguous fp32 tensor")
    if y is not None and (y.shape != x.shape or y.dtype != torch.float32):
        raise ValueError("add_dyt: the sublayer output must be fp32 of the stream's shape")
    if out is None and act_dtype is not None:
        out = torch.empty(T, d, dtype=act_dtype, device=x.device)
    if out is not None and (out.shape != x.shape or out.stride(1) != 1):
        raise ValueError("add_dyt: the output is a [T, d] block with unit column stride")
    if not x.is_cuda:
        ref.add_dyt(x, y, mult, alpha, w, b, out)
        return out
    if y is None and out is None:
        return None
    _hip().call("lc_add_dyt", x.data_ptr(), _hip().ptr(y.contiguous() if y is not None else None), float(mult), float(alpha),
                _hip().ptr(w), _hip().ptr(b), _hip().ptr(out), _f32flag(out.dtype) if out is not None else 0,
                max(out.stride(0), d) if out is not None else d, T, d)
    return out


def rope_pairs_write(qk: torch.Tensor, inv_freq: Optional[torch.Tensor], positions: torch.Tensor, slot_mapping: torch.Tensor,
                     k_cache: torch.Tensor, v_cache: Optional[torch.Tensor], H: int, G: int, D: int, rot_dims: int) -> torch.Tensor:
    """Attention pre-processing of a layer without norms or biases whose values are its keys: qk fp32
    [T, >= (H + G) D] = q | k; the first ``rot_dims`` coordinates of each head rotate in neighbouring pairs
    (2i, 2i + 1) by position * inv_freq[i] (``inv_freq`` fp64 [rot_dims / 2]); rotated keys are written to
    ``k_cache`` [blocks, G, BS, D] and the keys as projected to ``v_cache`` (None when nothing rotates and one
    plane is both). Returns the rotated q fp32 [T, H*D]."""
    if rot_dims and (inv_freq is None or inv_freq.dtype != torch.float64 or inv_freq.numel() != rot_dims // 2 or v_cache is None):
        raise ValueError("rope_pairs_write: rot_dims / 2 fp64 frequencies and a value plane are needed")
    if k_cache.shape[1:] != (G, k_cache.shape[2], D) or (v_cache is not None and v_cache.shape != k_cache.shape):
        raise ValueError("rope_pairs_write: cache planes do not fit the head sizes")
    if not qk.is_cuda:
        return ref.rope_pairs_write(qk, inv_freq, positions, slot_mapping, k_cache, v_cache, H, G, D, rot_dims)
    T = qk.shape[0]
    if qk.dtype != torch.float32 or qk.stride(1) != 1 or qk.shape[1] < (H + G) * D:
        raise ValueError("rope_pairs_write: fp32 projections q | k")
    q = torch.empty(T, H * D, dtype=torch.float32, device=qk.device)
    _hip().call("lc_rope_pairs_write", qk.data_ptr(), qk.stride(0), _hip().ptr(inv_freq), positions.data_ptr(),
                slot_mapping.data_ptr(), k_cache.data_ptr(), _hip().ptr(v_cache), _f32flag(k_cache.dtype), q.data_ptr(),
                T, H, G, D, k_cache.shape[2], rot_dims)
    return q


def glu_clamped(y: torch.Tensor, col_gate: int, col_up: int, n: int, limit: float, act_dtype: torch.dtype,
                slot_of: Optional[torch.Tensor] = None, wts: Optional[torch.Tensor] = None, slope: float = 1.702,
                shift: float = 1.0) -> torch.Tensor:
    """Clamped gated unit over column blocks of an fp32 matrix y: g = min(s * y[:, col_gate:+n], limit),
    u = clamp(s * y[:, col_up:+n], -limit, limit), result g * sigmoid(slope * g) * (u + shift) in
    ``act_dtype`` [rows of y, n]. With ``slot_of`` / ``wts`` (int32 / fp32, one entry per (token, choice)
    pair) entry r names row slot_of[r] and its scale s = wts[r]: the expert-sorted rows of a routed
    feed-forward whose weight multiplies the expert's input."""
    R = y.shape[0]
    rows = slot_of.numel() if slot_of is not None else R
    if not y.is_cuda:
        return ref.glu_clamped(y, col_gate, col_up, n, limit, slope, shift, slot_of, wts, act_dtype, rows)
    if y.dtype != torch.float32 or y.stride(1) != 1 or max(col_gate, col_up) + n > y.shape[1]:
        raise ValueError("glu_clamped: an fp32 matrix holding both column blocks")
    if slot_of is not None and rows > R:
        raise ValueError("glu_clamped: more work entries than rows")
    out = torch.empty(R, n, dtype=act_dtype, device=y.device)
    _hip().call("lc_glu_clamped", y.data_ptr(), y.stride(0) if R > 1 else max(y.stride(0), y.shape[1]), int(col_gate),
                int(col_up), int(n), float(limit), float(slope), float(shift), _hip().ptr(slot_of), _hip().ptr(wts),
                out.data_ptr(), _f32flag(act_dtype), rows)
    return out


# ---- parallel residual streams, rotary values, mixed heads' weights, rotated latent keys, xIELU (hybrid_streams.hip) ----
MAX_STREAMS = 8


def hc_init(x0: torch.Tensor, w: torch.Tensor, eps: float, streams: int) -> torch.Tensor:
    """The start of a residual of several parallel streams: fp32 [T, S, d], every stream the RMS norm of x0
    (fp32 [T, d]) times w."""
    T, d = x0.shape
    if x0.dtype != torch.float32 or not x0.is_contiguous() or w.numel() != d or not 1 <= streams <= MAX_STREAMS:
        raise ValueError(f"hc_init: a contiguous fp32 matrix, a weight per column, 1..{MAX_STREAMS} streams")
    if not x0.is_cuda:
        return ref.hc_init(x0, w, eps, streams)
    xs = torch.empty(T, streams, d, dtype=torch.float32, device=x0.device)
    _hip().call("lc_hc_init", x0.data_ptr(), w.data_ptr(), float(eps), xs.data_ptr(), T, streams, d)
    return xs


def hc_step(xs: torch.Tensor, y: Optional[torch.Tensor], mix: Optional[torch.Tensor], out_w: Optional[torch.Tensor],
            in_w: Optional[torch.Tensor], norm_w: Optional[torch.Tensor], eps: float,
            act_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """One launch between two sublayers of a residual of S parallel streams xs (fp32 [T, S, d], in place). With
    ``y`` (fp32 [T, d], the sublayer's result): every new stream is a mixture of the old ones plus its share of
    y, xs[:, j] <- sum_s mix[s, j] xs[:, s] + out_w[j] y. With ``in_w``: the next sublayer's input
    u = sum_s in_w[s] xs[:, s]; returned RMS-normed times ``norm_w`` in ``act_dtype``, or, without a norm weight,
    as it is in fp32. Without ``in_w`` nothing is returned."""
    T, S, d = xs.shape
    if xs.dtype != torch.float32 or not xs.is_contiguous() or S > MAX_STREAMS:
        raise ValueError(f"hc_step: the streams are a contiguous fp32 [T, S, d] tensor, S <= {MAX_STREAMS}")
    if y is not None and (y.shape != (T, d) or y.dtype != torch.float32 or mix is None or out_w is None
                          or mix.numel() != S * S or out_w.numel() != S):
        raise ValueError("hc_step: an fp32 [T, d] result with mix [S, S] and out [S]")
    if (in_w is not None and in_w.numel() != S) or (norm_w is not None and (in_w is None or norm_w.numel() != d)):
        raise ValueError("hc_step: in [S], and a norm weight per column only with it")
    for c in (mix, out_w, in_w, norm_w):
        if c is not None and (c.dtype != torch.float32 or not c.is_contiguous()):
            raise ValueError("hc_step: fp32 coefficients")
    if not xs.is_cuda:
        return ref.hc_step(xs, y, mix, out_w, in_w, norm_w, eps, act_dtype)
    if y is None and in_w is None:
        return None
    u = torch.empty(T, d, dtype=torch.float32, device=xs.device) if in_w is not None and norm_w is None else None
    xa = torch.empty(T, d, dtype=act_dtype, device=xs.device) if norm_w is not None else None
    _hip().call("lc_hc_step", xs.data_ptr(), _hip().ptr(y.contiguous() if y is not None else None), _hip().ptr(mix),
                _hip().ptr(out_w), _hip().ptr(in_w), _hip().ptr(norm_w), float(eps), _hip().ptr(u), _hip().ptr(xa),
                _f32flag(act_dtype) if xa is not None else 0, T, S, d)
    return xa if xa is not None else u


def rope_qkv_write(qkv: torch.Tensor, inv_freq: Optional[torch.Tensor], inv_freq_v: Optional[torch.Tensor],
                   positions: torch.Tensor, slot_mapping: torch.Tensor, k_cache: Optional[torch.Tensor],
                   v_cache: Optional[torch.Tensor], H: int, G: int, D: int, Dv: int, rot_dims: int, pairs: bool = False,
                   v_pairs: bool = False) -> torch.Tensor:
    """Rotary positions and the paged cache write of an attention layer with a value projection: qkv fp32
    [T, >= H D + G (D + Dv)] = q | k | v. The first ``rot_dims`` coordinates of every query and key head turn by
    position * inv_freq[i] (fp64 [rot_dims / 2]); ``pairs``: neighbours (2i, 2i + 1) turn together, otherwise i
    with i + rot_dims / 2. With ``inv_freq_v`` (fp64 [Dv / 2]) every value head turns over its whole width by its
    own position (layout ``v_pairs``) and is cached so. Keys go to ``k_cache`` [blocks, G, BS, D], values to
    ``v_cache`` [blocks, G, BS, Dv]. Returns the turned q fp32 [T, H*D]."""
    if rot_dims and (inv_freq is None or inv_freq.dtype != torch.float64 or inv_freq.numel() != rot_dims // 2):
        raise ValueError("rope_qkv_write: rot_dims / 2 fp64 frequencies are needed")
    if inv_freq_v is not None and (inv_freq_v.dtype != torch.float64 or inv_freq_v.numel() * 2 != Dv):
        raise ValueError("rope_qkv_write: Dv / 2 fp64 frequencies for the values")
    if k_cache is not None and (k_cache.shape[1:] != (G, k_cache.shape[2], D) or v_cache.shape[1:] != (G, k_cache.shape[2], Dv)
                                or not k_cache.is_contiguous() or not v_cache.is_contiguous() or k_cache.dtype != v_cache.dtype):
        raise ValueError("rope_qkv_write: cache planes do not fit the head sizes")
    if qkv.dtype != torch.float32 or qkv.stride(1) != 1 or qkv.shape[1] < H * D + G * (D + Dv):
        raise ValueError("rope_qkv_write: fp32 projections q | k | v")
    if not qkv.is_cuda:
        return ref.rope_qkv_write(qkv, inv_freq, inv_freq_v, positions, slot_mapping, k_cache, v_cache, H, G, D, Dv,
                                  rot_dims, pairs, v_pairs)
    T = qkv.shape[0]
    q = torch.empty(T, H * D, dtype=torch.float32, device=qkv.device)
    _hip().call("lc_rope_qkv_write", qkv.data_ptr(), max(qkv.stride(0), qkv.shape[1]), _hip().ptr(inv_freq),
                _hip().ptr(inv_freq_v), positions.data_ptr(), slot_mapping.data_ptr(), _hip().ptr(k_cache), _hip().ptr(v_cache),
                _f32flag(k_cache.dtype) if k_cache is not None else 0, q.data_ptr(), T, H, G, D, Dv,
                k_cache.shape[2] if k_cache is not None else 1, rot_dims, 1 if pairs else 0, 1 if v_pairs else 0)
    return q


def talk_mix(o: torch.Tensor, talk: torch.Tensor, positions: torch.Tensor, inv_freq_v: Optional[torch.Tensor], H: int,
             G: int, Dv: int, act_dtype: torch.dtype, v_pairs: bool = False) -> torch.Tensor:
    """The heads' softmax weights mixed by ``talk`` (fp32 [H, H]: new head h = sum_g talk[h, g] head g), applied
    behind the weighted sums: o fp32 [T, H * G * Dv] holds every head's weights on every value head
    (``attn_masked(..., all_value_heads=True)``); out[t, h] = sum_g talk[h, g] o[t, g, h / (H / G)]. With
    ``inv_freq_v`` (fp64 [Dv / 2]) each head's result turns back by its row's position over its whole width.
    Returns [T, H * Dv] in ``act_dtype``."""
    T = o.shape[0]
    if o.dtype != torch.float32 or not o.is_contiguous() or o.shape[1] != H * G * Dv or talk.numel() != H * H or \
            talk.dtype != torch.float32 or not talk.is_contiguous() or H % G:
        raise ValueError("talk_mix: fp32 sums [T, H * G * Dv] and an fp32 [H, H] mixing matrix")
    if inv_freq_v is not None and (inv_freq_v.dtype != torch.float64 or inv_freq_v.numel() * 2 != Dv):
        raise ValueError("talk_mix: Dv / 2 fp64 frequencies")
    if not o.is_cuda:
        return ref.talk_mix(o, talk, positions, inv_freq_v, H, G, Dv, act_dtype, v_pairs)
    out = torch.empty(T, H * Dv, dtype=act_dtype, device=o.device)
    _hip().call("lc_talk_mix", o.data_ptr(), talk.data_ptr(), positions.data_ptr(), _hip().ptr(inv_freq_v), out.data_ptr(),
                _f32flag(act_dtype), T, H, G, Dv, 1 if v_pairs else 0)
    return out


def latent_rope_write(proj: torch.Tensor, col_c: int, w: Optional[torch.Tensor], eps: float, inv_freq: Optional[torch.Tensor],
                      positions: torch.Tensor, slot_mapping: torch.Tensor, cache: Optional[torch.Tensor], qlat: torch.Tensor,
                      H: int, D: int, R: int, rd: int, pairs: bool = True) -> None:
    """Latent attention whose cached row carries a rotated key part that all heads share. proj fp32 [T, ...]:
    queries from column 0, head by head [D plain | rd to turn]; with ``cache`` ([blocks, 1, BS, R + rd]) also the
    compressed row and the shared key part, R + rd columns from ``col_c`` on: the cache row at the token's slot
    becomes rms_norm(compressed) * w | turned key part. The turned query parts go to columns R .. R + rd - 1 of each
    head's block of ``qlat`` (fp32 [T, H * (R + rd)]). ``inv_freq`` fp64 [rd / 2]; ``pairs``: neighbours turn together."""
    T = proj.shape[0]
    if proj.dtype != torch.float32 or proj.stride(1) != 1 or proj.shape[1] < H * (D + rd):
        raise ValueError("latent_rope_write: fp32 projections")
    if qlat.shape != (T, H * (R + rd)) or qlat.dtype != torch.float32 or not qlat.is_contiguous():
        raise ValueError("latent_rope_write: queries in the cached row's coordinates are fp32 [T, H * (R + rd)]")
    if rd and (rd % 2 or inv_freq is None or inv_freq.dtype != torch.float64 or inv_freq.numel() != rd // 2):
        raise ValueError("latent_rope_write: rd / 2 fp64 frequencies are needed")
    if cache is not None and (cache.shape[1] != 1 or cache.shape[3] != R + rd or not cache.is_contiguous() or w is None
                              or w.numel() != R or col_c < H * (D + rd) or col_c + R + rd > proj.shape[1]):
        raise ValueError("latent_rope_write: a one-head cache plane of width R + rd and the compressed row's columns")
    if not proj.is_cuda:
        return ref.latent_rope_write(proj, col_c, w, eps, inv_freq, positions, slot_mapping, cache, qlat, H, D, R, rd, pairs)
    _hip().call("lc_latent_rope_write", proj.data_ptr(), max(proj.stride(0), proj.shape[1]), int(col_c), _hip().ptr(w),
                float(eps), _hip().ptr(inv_freq), positions.data_ptr(), slot_mapping.data_ptr(), _hip().ptr(cache),
                _f32flag(cache.dtype) if cache is not None else 0, qlat.data_ptr(), T, H, D, R, rd,
                cache.shape[2] if cache is not None else 1, 1 if pairs else 0)


def xielu(y: torch.Tensor, ap: float, an: float, act_dtype: torch.dtype) -> torch.Tensor:
    """xIELU of an fp32 matrix (may be a column slice): ap z^2 + z / 2 above zero, an (exp(z) - 1 - z) + z / 2 at
    and below it, in ``act_dtype``."""
    if not y.is_cuda:
        return ref.xielu(y, ap, an, act_dtype)
    if y.dim() != 2 or y.stride(1) != 1 or y.dtype != torch.float32:
        raise ValueError("xielu: an fp32 matrix with unit column stride")
    T, n = y.shape
    out = torch.empty(T, n, dtype=act_dtype, device=y.device)
    _hip().call("lc_xielu", y.data_ptr(), max(y.stride(0), n), out.data_ptr(), _f32flag(act_dtype), T, n, float(ap), float(an))
    return out
