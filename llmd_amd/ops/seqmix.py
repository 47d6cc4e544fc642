"""Ops of per-layer ("sequence mixer") stacks: latent attention of any size, the selective
scan, the generalized delta rule, zero-centred norms with layer scale, depth averaging, plain
(ungated) expert feed-forwards; hyper-connected residual streams with layer norm, grouped-query
attention with its own key and value sizes (bias, rotary, unit norm, value mixing, gate), gated
activations, score routing with a selection-only correction, gated experts with identity experts;
the bigram embedding, the post-norm residual add, the gated delta rule, distance slopes / chunks /
sinks in grouped attention, sigmoid routing with experts whose weight scales their input; the embedding
with the first norm, plain RMS norms of projections, the input convolution, the squared ReLU, the
HGRN2 recurrence, sliding windows with kept first tokens, keys as values, per-head gates of latent
attention.

GPU tensors go to the ``llmd_amd._C_seqmix`` library (csrc/seqmix/*.hip, built on its own so a
model that needs only these kernels compiles only these); it is templated on the activation
type, bfloat16 or float32, and keeps in fp32 what the recurrences, norms, scores and the
residual need. CPU tensors use ``seqmix_ref``. A missing library on a GPU host raises.

Step layout (engine/attn_meta.py SeqMeta): the step's tokens are the sequences' runs back to
back; ``seq_start`` [n+1] bounds them, ``seq_slot`` [n] is each sequence's state slot and
``seq_init`` [n] says whether the slot holds the sequence's earlier state (0: start from zero).
"""
from __future__ import annotations

import importlib
import os

import torch

from . import seqmix_ref as ref

_LIB = None


def native():
    global _LIB
    if _LIB is None:
        try:
            _LIB = importlib.import_module("llmd_amd._C_seqmix")
        except ImportError as e:
            if os.environ.get("LLMD_AUTOBUILD", "1") != "1":
                raise RuntimeError(f"llmd_amd._C_seqmix HIP extension not built: {e}") from e
            from llmd_amd.build import build_seqmix

            build_seqmix()
            _LIB = importlib.import_module("llmd_amd._C_seqmix")
    return _LIB


def embed_scale(ids, table, scale: float, hist):
    """hist[0] = hist[1] = table[ids] * scale (fp32): the embedding output and the first layer's
    working residual."""
    if not ids.is_cuda:
        return ref.embed_scale(ids, table, scale, hist)
    native().embed_scale(ids, table, float(scale), hist)


def zc_norm(x, w, eps: float, out_dtype):
    """RMS norm of the fp32 residual with a weight stored around zero: x / rms(x) * (1 + w)."""
    if not x.is_cuda:
        return ref.zc_norm(x, w, eps, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    native().zc_norm(x, w, float(eps), out)
    return out


def add_post_norm(y, w_post, ls, x, eps: float, next_w=None, out_dtype=None):
    """x += ls * zc_norm(y, w_post) on the fp32 residual, in place; with ``next_w`` also returns
    zc_norm(x, next_w), the next sublayer's input, from the same pass."""
    if not x.is_cuda:
        return ref.add_post_norm(y, w_post, ls, x, eps, next_w, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device) if next_w is not None else None
    native().add_post_norm(y, w_post, ls, x, float(eps), next_w, out)
    return out


def depth_avg_norm(hist, n: int, coef, dst: int, norm_w, eps: float, out_dtype):
    """hist[dst] = sum_{j<n} coef[j] * hist[j] (fp32) and the zero-centred norm of that sum."""
    if not hist.is_cuda:
        return ref.depth_avg_norm(hist, n, coef, dst, norm_w, eps, out_dtype)
    out = torch.empty(hist.shape[1:], dtype=out_dtype, device=hist.device)
    native().depth_avg_norm(hist, int(n), coef, int(dst), norm_w, float(eps), out)
    return out


def latent_rope_cache(q, kv, norm_w, eps, positions, cos_sin, H, dn, dr, rot_dims, R, slots, cache, q_abs,
                      interleaved: bool = False):
    """Rotate the rotary part of q into ``q_abs[..., R:]``; write [norm(kv[:, :R]) | rot(kv[:, R:])]
    to the paged latent cache at ``slots`` (-1: no write). cos_sin [max_pos, rot_dims] fp32; pairs
    (i, i + rot_dims/2), or (2i, 2i+1) when ``interleaved``. ``kv`` None: a layer that reads another
    layer's cache rotates its queries only."""
    if not q.is_cuda:
        return ref.latent_rope_cache(q, kv, norm_w, eps, positions, cos_sin, H, dn, dr, rot_dims, R, slots, cache,
                                     q_abs, interleaved)
    native().latent_rope_cache(q, kv, norm_w, float(eps), positions, cos_sin, H, dn, dr, rot_dims, R, slots, cache,
                               q_abs, bool(interleaved))


MFMA_ATTENTION = os.environ.get("LLMD_LATENT_MFMA", "1") == "1"


def latent_attention(q_abs, cache, tables, row_seq, row_len, scale: float, R: int, rows_per_group: int = 1,
                     seq=None, gate=None):
    """Causal softmax attention of absorbed queries [T, H, R + dr] over the paged latent cache
    [blocks, bs, R + dr]; row t sees the first row_len[t] keys of sequence row_seq[t].
    Returns the latent outputs [T, H, R]. ``gate`` [T, H] (a column view of a projection): head h's
    output is multiplied by sigmoid(gate[t, h]).

    bfloat16 with the step's ``seq`` description (engine/attn_meta.py SeqMeta): the matrix-core
    kernel over work items of up to 64 (token, head) rows of one sequence (R + dr <= 576, R <= 512,
    H <= 64). Otherwise (float32, other sizes) the fp32 FMA kernel; ``rows_per_group`` (1 or 4) is
    its number of consecutive rows that share a workgroup's key tiles."""
    T, H, _ = q_abs.shape
    out = torch.empty(T, H, R, dtype=q_abs.dtype, device=q_abs.device)
    if not q_abs.is_cuda:
        return ref.latent_attention(q_abs, cache, tables, row_seq, row_len, scale, R, out, gate)
    if MFMA_ATTENTION and seq is not None and q_abs.dtype == torch.bfloat16 and H <= 64:
        items = seq.attention_items(max(1, 64 // H))
        nsplit, split, po, pm = 1, 0, None, None
        if seq.max_q == 1 and seq.max_len > 256:
            # decode-only step: cut the keys into ranges so that items x ranges fill the chip
            n = items.shape[0]
            nsplit = max(1, min(-(-512 // n), seq.max_len // 128))
            split = -(-seq.max_len // (nsplit * 32)) * 32
            nsplit = -(-seq.max_len // split)
            if nsplit > 1:
                po = torch.empty(n * nsplit * 64 * R, dtype=torch.float32, device=q_abs.device)
                pm = torch.empty(n * nsplit * 128, dtype=torch.float32, device=q_abs.device)
        if native().latent_attention_mfma(q_abs, cache, tables, items, row_len, float(scale), R, out, nsplit, split,
                                          po, pm, gate):
            return out
    native().latent_attention(q_abs, cache, tables, row_seq, row_len, float(scale), R, int(rows_per_group), out, gate)
    return out


def causal_conv_silu(xz, C, w, b, conv_state, seq_start, seq_slot, seq_init, max_q: int):
    """Per-channel causal convolution + SiLU over the first C columns of xz, continuing from each
    sequence's last taps-1 inputs in ``conv_state`` [slots, taps-1, C] (updated). ``max_q``: the
    longest run of the step (sizes the grid)."""
    out = torch.empty(xz.shape[0], C, dtype=xz.dtype, device=xz.device)
    if not xz.is_cuda:
        return ref.causal_conv_silu(xz, C, w, b, conv_state, seq_start, seq_slot, seq_init, out)
    native().causal_conv_silu(xz, C, w, b, conv_state, seq_start, seq_slot, seq_init, int(max_q), out)
    return out


def selective_scan(xc, dt_raw, dt_bias, A, bc, R, N, D, xz, C, state, seq_start, seq_slot, seq_init):
    """S <- exp(dt A) S + dt x B; y = S C + D x; y * silu(z). dt = softplus(dt_raw + dt_bias);
    B, C are columns [R, R+N) and [R+N, R+2N) of ``bc``; z the columns [C, 2C) of xz. ``state``
    [slots, C, N] fp32 is continued and updated."""
    out = torch.empty_like(xc)
    if not xc.is_cuda:
        return ref.selective_scan(xc, dt_raw, dt_bias, A, bc, R, N, D, xz, C, state, seq_start, seq_slot, seq_init,
                                  out)
    native().selective_scan(xc, dt_raw, dt_bias, A, bc, R, N, D, xz, C, state, seq_start, seq_slot, seq_init, out)
    return out


def gdelta_scan(proj, wl, w0, a_b, norm_w, eps, H, d, state, seq_start, seq_slot, seq_init):
    """Generalized delta rule over ``proj`` = [r | k | v | g | a] (H*d columns each) with decay
    logits ``wl``: S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r, then per-head RMS norm,
    ``norm_w`` and the sigmoid gate. ``state`` [slots, H, d, d] fp32."""
    out = torch.empty(proj.shape[0], H * d, dtype=proj.dtype, device=proj.device)
    if not proj.is_cuda:
        return ref.gdelta_scan(proj, wl, w0, a_b, norm_w, eps, H, d, state, seq_start, seq_slot, seq_init, out)
    native().gdelta_scan(proj, wl, w0, a_b, norm_w, float(eps), H, d, state, seq_start, seq_slot, seq_init, out)
    return out


def xielu(z, ap: float, aq: float):
    """z > 0: ap z^2 + z/2; else aq (exp(z) - 1 - z) + z/2."""
    if not z.is_cuda:
        return ref.xielu(z, ap, aq)
    out = torch.empty_like(z)
    native().xielu(z, float(ap), float(aq), out)
    return out


def moe_route(logits, k: int, sigmoid: bool = False):
    """Top-k of fp32 router logits (ties: lower index) and the softmax over the chosen ones; with
    ``sigmoid`` the weights are the chosen logits' sigmoids instead, each on its own (the largest
    sigmoid scores are the largest logits)."""
    if not logits.is_cuda:
        return ref.moe_route(logits, k, sigmoid)
    T = logits.shape[0]
    ids = torch.empty(T, k, dtype=torch.int32, device=logits.device)
    w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    native().moe_route(logits, k, ids, w, bool(sigmoid))
    return ids, w


MOE_TILE = 64


def moe_ffn(h, ids, w, w1, w2):
    """sum_j w[t, j] * W2[e] gelu(W1[e] h_t), e = ids[t, j]: ungated experts with the exact (erf)
    GELU. w1 [E, F, d], w2 [E, d, F]. Rows are grouped by expert into 64-row tiles (one pass of a
    single workgroup), two grouped GEMMs run over the tiles, and the combine sums each token's
    rows in fp32; a row's sums do not depend on what else is in the step."""
    if not h.is_cuda:
        return ref.moe_ffn(h, ids, w, w1, w2)
    C = native()
    T, d = h.shape
    k = ids.shape[1]
    E, Fh, _ = w1.shape
    n = T * k
    max_tiles = (n + E * (MOE_TILE - 1)) // MOE_TILE + 1
    dev = h.device
    slot_row = torch.empty(max_tiles * MOE_TILE, dtype=torch.int32, device=dev)   # tile slot -> pair index or -1
    tile_e = torch.empty(max_tiles, dtype=torch.int32, device=dev)                # tile -> expert or -1
    pair_slot = torch.empty(n, dtype=torch.int32, device=dev)                      # pair -> tile slot
    C.moe_group(ids, E, slot_row, tile_e, pair_slot)
    a = torch.empty(max_tiles * MOE_TILE, Fh, dtype=h.dtype, device=dev)
    y = torch.empty(max_tiles * MOE_TILE, d, dtype=h.dtype, device=dev)
    C.moe_gemm(h, k, slot_row, tile_e, w1, a, 1, n, None)   # n = rows of the step: picks the tile width
    C.moe_gemm(a, 0, slot_row, tile_e, w2, y, 0, n, None)
    out = torch.empty_like(h)
    C.moe_combine(y, pair_slot, w, out, None)
    return out


# ---- hyper-connected residual streams
def hyper_embed(ids, table, X):
    """X[s] = table[ids] for every stream s (fp32 [S, T, d])."""
    if not ids.is_cuda:
        return ref.hyper_embed(ids, table, X)
    native().hyper_embed(ids, table, X)


def hyper_norm(X, w_in, norm_w, eps: float, out_dtype):
    """Layer norm (weight, no bias; two-pass fp32 variance) of u = sum_s w_in[s] X[s]."""
    if not X.is_cuda:
        return ref.hyper_norm(X, w_in, norm_w, eps, out_dtype)
    out = torch.empty(X.shape[1:], dtype=out_dtype, device=X.device)
    native().hyper_norm(X, w_in, norm_w, float(eps), out)
    return out


def hyper_update_norm(X, y, mix, w_out, next_in=None, next_w=None, eps: float = 0.0, out_dtype=None):
    """X[t] <- sum_s mix[s, t] X[s] + w_out[t] y for all streams at once, in place (fp32); with
    ``next_w`` also returns the layer norm of sum_s next_in[s] X[s], the next sublayer's input (or
    the model's final norm over the plain sum), from the same pass."""
    if not X.is_cuda:
        return ref.hyper_update_norm(X, y, mix, w_out, next_in, next_w, eps, out_dtype)
    out = torch.empty(X.shape[1:], dtype=out_dtype, device=X.device) if next_w is not None else None
    native().hyper_update_norm(X, y, mix, w_out, next_in, next_w, float(eps), out)
    return out


# ---- grouped-query attention with its own key and value sizes
def qkv_rope_cache(qkv, bias, positions, cos_sin, Hq, Hkv, dim, vdim, rot_dims, interleaved, unit_eps, v_first,
                   v_mode, lam, slots, cache, q_out, qk_w=None, norm_first: bool = False, v_from_k: bool = False):
    """From a fused projection [q | k | v | ...] of a step's tokens: add ``bias`` (fp32, over q|k|v),
    rotate the first ``rot_dims`` dimensions of every query and key head by the angles of ``cos_sin``
    [max_pos, rot_dims] = [cos | sin] (pairs (2i, 2i+1) when ``interleaved``, (i, i + rot_dims/2)
    otherwise), divide each head by its root mean square (``unit_eps`` not None), mix the values with
    those of an earlier layer (``v_mode`` 1: store this layer's values in ``v_first`` fp32
    [T, Hkv * vdim]; 2: v <- (1 - lam) v + lam v_first), write queries to ``q_out`` [T, Hq, dim] and
    the row [key | value] of every kv head to the paged ``cache`` [blocks, Hkv, bs, dim + vdim] at
    ``slots`` (-1: no write). ``qk_w`` fp32 [2, dim]: weights of the query and of the key norm (with
    ``unit_eps``), shared by the heads. ``bias`` may be None. All arithmetic fp32.
    ``norm_first``: the division by the root mean square and the weights come before the rotation.
    ``v_from_k``: the projection is [q | k | ...] and the values are its keys (with their bias), as
    projected - before norm and rotation (vdim == dim)."""
    if not qkv.is_cuda:
        return ref.qkv_rope_cache(qkv, bias, positions, cos_sin, Hq, Hkv, dim, vdim, rot_dims, interleaved, unit_eps,
                                  v_first, v_mode, lam, slots, cache, q_out, qk_w, norm_first, v_from_k)
    native().qkv_rope_cache(qkv, bias, positions, cos_sin, Hq, Hkv, dim, vdim, rot_dims, bool(interleaved),
                            unit_eps is not None, float(unit_eps or 0.0), v_first, int(v_mode), float(lam), slots, cache,
                            q_out, qk_w, bool(norm_first), bool(v_from_k))


GQA_MFMA = os.environ.get("LLMD_GQA_MFMA", "1") == "1"
GQA_DECODE_WGS = int(os.environ.get("LLMD_GQA_DECODE_WGS", "2048"))  # workgroups a decode-only step aims for
# ... and with a sliding window: a row's keys are few, so a range's fixed work (query fragments, partial
# results, the merge) weighs more. 64 sequences x 8 kv heads, window 1024 at context 2048, ms per layer of
# the whole stack: 0.225 / 0.247 / 0.263 / 0.287 for 512 / 1024 / 2048 / 4096
GQA_WINDOW_DECODE_WGS = int(os.environ.get("LLMD_GQA_WINDOW_DECODE_WGS", "512"))
# LLMD_GQA_RB2=1: prompt portions run as 128-row items, two blocks of 16 rows per wave. Measured slower
# than 64-row items at 128/128 heads (2048-token prompt: 227 us against 181 us - 185 + 64 registers
# leave two waves per SIMD instead of three), so it stays an option.
GQA_RB2 = os.environ.get("LLMD_GQA_RB2", "0") == "1"


def grouped_attention(q, cache, dim, vdim, scale: float, seq, gate=None, slopes=None, chunk: int = 0, sinks=None,
                      window: int = 0, keep_first: int = 0):
    """Causal softmax attention of q [T, Hq, dim] over the paged cache [blocks, Hkv, bs, dim + vdim]
    (query head h reads kv head h // (Hq / Hkv)); row t sees the first seq.row_len[t] keys of its
    sequence. ``gate`` [T, Hq * vdim] (a column view of the fused projection): the result is
    multiplied by sigmoid(gate). Returns [T, Hq * vdim].

    ``slopes`` fp32 [Hq]: the score of query i and key j loses slopes[h] * (i - j).
    ``chunk`` > 0: query i sees key j only inside its own chunk, j >= (i // chunk) * chunk; i and j are
    positions in the sequence, not in the step.
    ``sinks`` fp32 [Hq]: one more score per head in the softmax's denominator, without a value.
    ``window`` > 0: query i sees key j <= i only if i - j < window or j < ``keep_first`` (positions in
    the sequence); key tiles that lie between the kept first tokens and the window are not visited.

    bfloat16 runs on the matrix cores (work item = up to 64 (token, head-of-group) rows of one
    sequence and kv head); float32 and sizes outside the compiled forms on the fp32 FMA kernel."""
    T, Hq, _ = q.shape
    Hkv = cache.shape[1]
    out = torch.empty(T, Hq * vdim, dtype=q.dtype, device=q.device)
    if not q.is_cuda:
        return ref.grouped_attention(q, cache, dim, vdim, seq.tables, seq.row_seq, seq.row_len, scale, gate, out,
                                     slopes, chunk, sinks, window, keep_first)
    G = Hq // Hkv
    chunk, window = int(chunk), int(window)
    keep_first = int(keep_first) if window else 0
    if window and chunk:
        raise ValueError("a sliding window and chunks do not combine")
    # keys a row can see at most: with chunks, its chunk (and the tile that the chunk starts in); with a
    # window, the tiles of the kept first tokens and those of the window
    span = min(seq.max_len, chunk + 32) if chunk else seq.max_len
    if window:
        span = min(seq.max_len, -(-keep_first // 32) * 32 + window + 32)
    if GQA_MFMA and q.dtype == torch.bfloat16 and G <= 64:
        rb = 2 if GQA_RB2 and seq.max_q * G > 64 else 1
        # workgroup ids run over the kv heads first: ids 256 apart (256 // Hkv items apart) share a CU
        items = seq.attention_items(max(1, 64 * rb // G), balance=max(1, 256 // Hkv) if seq.max_q > 1 else 0)
        nsplit, split, po, pm = 1, 0, None, None
        if seq.max_q == 1 and span > 256:
            # decode-only step: key ranges so that items x kv heads x ranges give the chip about
            # eight workgroups per CU (a workgroup walks its tiles one after another)
            n = items.shape[0] * Hkv
            nsplit = max(1, min(-(-(GQA_WINDOW_DECODE_WGS if window else GQA_DECODE_WGS) // n), span // 128))
            split = -(-span // (nsplit * 32)) * 32
            nsplit = -(-span // split)
            if nsplit > 1:
                po = torch.empty(n * nsplit * 64 * vdim, dtype=torch.float32, device=q.device)
                pm = torch.empty(n * nsplit * 128, dtype=torch.float32, device=q.device)
        if native().grouped_attention_mfma(q, cache, dim, vdim, seq.tables, items, seq.row_len, float(scale), gate,
                                           out, nsplit, split, po, pm, rb, slopes, chunk, sinks, window, keep_first):
            return out
    native().grouped_attention(q, cache, dim, vdim, seq.tables, seq.row_seq, seq.row_len, float(scale), gate,
                               4 if seq.max_q > 1 else 1, out, slopes, chunk, sinks, window, keep_first)
    return out


ACT_KINDS = {"gelu_tanh": 0, "silu": 1}


def gated_act(gu, Fh: int, kind: str):
    """act(gu[:, :Fh]) * gu[:, Fh:], act the tanh form of GELU or SiLU, fp32 arithmetic."""
    if not gu.is_cuda:
        return ref.gated_act(gu, Fh, kind)
    out = torch.empty(gu.shape[0], Fh, dtype=gu.dtype, device=gu.device)
    native().gated_act(gu, int(Fh), ACT_KINDS[kind], out)
    return out


def moe_route_scores(logits, correction, k: int):
    """Scores = softmax over ALL router outputs (fp32); the k largest of score + correction are
    chosen (ties: lower index); weights = the chosen scores / (their sum + 1e-20)."""
    if not logits.is_cuda:
        return ref.moe_route_scores(logits, correction, k)
    T = logits.shape[0]
    ids = torch.empty(T, k, dtype=torch.int32, device=logits.device)
    w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    native().moe_route_scores(logits, correction, k, ids, w)
    return ids, w


def moe_gated_ffn(h, ids, w, w1, w2, kind: str = "silu", scale_input: bool = False):
    """sum_j w[t, j] * W2[e] (act(Wg[e] h_t) * (Wu[e] h_t)), e = ids[t, j]; w1 [E, 2F, d] holds
    [gate rows | up rows], w2 [E, d, F]. ids >= E name identity experts: their output is h_t itself.
    Same grouping, tile GEMMs and fp32 combine as ``moe_ffn``; the activation and the product are the
    first GEMM's epilogue (a workgroup computes matching gate and up columns).

    ``scale_input``: the weight multiplies the expert's input instead of its output,
    sum_j W2[e] (act(Wg[e] (w h_t)) * (Wu[e] (w h_t))): the first GEMM's fp32 sums are scaled by the
    pair's weight before the activation (both products are linear in the input) and the combine adds
    the rows as they are. No identity experts in this form."""
    if not h.is_cuda:
        return ref.moe_gated_ffn(h, ids, w, w1, w2, kind, scale_input)
    C = native()
    T, d = h.shape
    k = ids.shape[1]
    E, F2, _ = w1.shape
    Fh = F2 // 2
    n = T * k
    max_tiles = (n + E * (MOE_TILE - 1)) // MOE_TILE + 1
    dev = h.device
    slot_row = torch.empty(max_tiles * MOE_TILE, dtype=torch.int32, device=dev)
    tile_e = torch.empty(max_tiles, dtype=torch.int32, device=dev)
    pair_slot = torch.empty(n, dtype=torch.int32, device=dev)       # -1: identity expert
    C.moe_group(ids, E, slot_row, tile_e, pair_slot)
    a = torch.empty(max_tiles * MOE_TILE, Fh, dtype=h.dtype, device=dev)
    y = torch.empty(max_tiles * MOE_TILE, d, dtype=h.dtype, device=dev)
    C.moe_gemm(h, k, slot_row, tile_e, w1, a, 2 + ACT_KINDS[kind], n, w if scale_input else None)
    C.moe_gemm(a, 0, slot_row, tile_e, w2, y, 0, n, None)
    out = torch.empty_like(h)
    C.moe_combine(y, pair_slot, None if scale_input else w, out, h)
    return out


def softcap_(logits, cap: float):
    """logits <- cap * tanh(logits / cap), in place (fp32)."""
    if not logits.is_cuda:
        return ref.softcap_(logits, cap)
    native().softcap(logits, float(cap))
    return logits


# ---- bigram embedding, post-norm residual, gated delta rule
def bigram_embed(ids, table, scale: float, bigram, buckets: int, mul_prev: int, mul_cur: int, prev_state, seq, x,
                 out_dtype):
    """x = table[ids] * scale + bigram[row] (fp32) and its copy in the activation type. The row of a
    token is (previous token * mul_prev + token * mul_cur) mod buckets, row ``buckets`` for a
    sequence's first token; the previous token of a run's first token is the sequence's state
    ``prev_state`` [slots, 1] int32 (read when seq_init is set; the run's last token is written
    back). ``bigram`` None: the scaled embedding alone."""
    if not ids.is_cuda:
        return ref.bigram_embed(ids, table, scale, bigram, buckets, mul_prev, mul_cur, prev_state, seq.seq_start,
                                seq.seq_slot, seq.seq_init, x, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    native().bigram_embed(ids, table, float(scale), bigram, int(buckets), int(mul_prev), int(mul_cur), prev_state,
                          seq.row_seq, seq.seq_start, seq.seq_slot, seq.seq_init, x, out)
    return out


def post_norm_add(y, w_post, x, eps: float, out_dtype, next_w=None, y2=None, a: float = 1.0, b: float = 1.0,
                  bias=None):
    """x += rms_norm(a y + b y2 + bias) * w_post on the fp32 residual, in place (plain weights, eps
    inside the root; ``y2`` and ``bias`` optional). Returns the next reader's input from the same
    pass: x in the activation type, or rms_norm(x) * next_w when ``next_w`` is given."""
    if not x.is_cuda:
        return ref.post_norm_add(y, w_post, x, eps, out_dtype, next_w, y2, a, b, bias)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    native().post_norm_add(y, y2, float(a), float(b), bias, w_post, x, float(eps), next_w, out)
    return out


def gated_delta_scan(xc, G: int, dk: int, H: int, dv: int, beta_raw, decay_raw, A, dt_bias, gate_raw,
                     gate_sigmoid: bool, norm_w, eps: float, state, seq):
    """Gated delta rule over a step's runs. ``xc`` [T, 2 G dk + H dv] = [q | k | v] after the short
    convolution and SiLU (G query/key heads of size dk, H value heads of size dv, value head h uses
    q/k head h // (H / G)). Per token and head, all fp32: q and k become unit vectors
    (x / sqrt(sum x^2 + 1e-6)), q times dk^-1/2; beta = sigmoid(beta_raw [T, H]); the decay is
    g = exp(-A_h softplus(decay_raw + dt_bias)), one per head (decay_raw [T, H]) or one per head and
    key channel (decay_raw [T, H dk], acting on the rows of S); then

        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q

    and o / rms(o) * norm_w [dv] * gate, gate = silu(gate_raw) or sigmoid(gate_raw) ([T, H dv]).
    ``state`` [slots, H, dk, dv] fp32 is continued (seq_init) and written back. beta_raw, decay_raw
    and gate_raw may be column views of one projection. Returns [T, H dv]."""
    out = torch.empty(xc.shape[0], H * dv, dtype=xc.dtype, device=xc.device)
    if not xc.is_cuda:
        return ref.gated_delta_scan(xc, G, dk, H, dv, beta_raw, decay_raw, A, dt_bias, gate_raw, gate_sigmoid, norm_w,
                                    eps, state, seq.seq_start, seq.seq_slot, seq.seq_init, out)
    native().gated_delta_scan(xc, int(G), int(dk), int(H), int(dv), beta_raw, decay_raw, A, dt_bias, gate_raw,
                              bool(gate_sigmoid), norm_w, float(eps), state, seq.seq_start, seq.seq_slot, seq.seq_init,
                              out)
    return out


# ---- embedding with the first norm, plain norms, input convolution, squared ReLU, HGRN2
def embed_norm(ids, table, w, eps: float, x, out_dtype):
    """x = table[ids] (the fp32 residual) and, from the same pass, rms_norm(x) * w in the activation type:
    the first sublayer's input of a stack that norms before its sublayers."""
    if not ids.is_cuda:
        return ref.embed_norm(ids, table, w, eps, x, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    native().embed_norm(ids, table, w, float(eps), x, out)
    return out


def rms_norm(y, w, eps: float):
    """y / sqrt(mean(y^2) + eps) * w over the rows of y [T, n] (a column view of a projection is
    fine), fp32 arithmetic, result in y's type."""
    if not y.is_cuda:
        return ref.rms_norm(y, w, eps)
    out = torch.empty(y.shape, dtype=y.dtype, device=y.device)
    native().rms_norm(y, w, float(eps), out)
    return out


def input_conv(h, w, state, seq):
    """h + conv(h) per channel over each sequence's run: conv(h)_t = sum_j w[:, j] h_(t - taps + 1 + j),
    continuing from the sequence's last taps - 1 inputs in ``state`` [slots, taps - 1, C] (read when
    seq_init is set, zeros otherwise; rolled forward to the run's end). ``seq.max_q`` is the step's
    longest run: a step of single tokens rolls the states in the same launch."""
    out = torch.empty_like(h)
    if not h.is_cuda:
        return ref.input_conv(h, w, state, seq.seq_start, seq.seq_slot, seq.seq_init, out)
    native().input_conv(h, w, state, seq.row_seq, seq.seq_start, seq.seq_slot, seq.seq_init, int(seq.max_q), out)
    return out


def relu2(z):
    """max(z, 0)^2."""
    if not z.is_cuda:
        return ref.relu2(z)
    out = torch.empty_like(z)
    native().relu2(z, out)
    return out


HGRN2_CHUNKED = os.environ.get("LLMD_HGRN2_CHUNKED", "1") == "1"
HGRN2_CHUNK_FROM = int(os.environ.get("LLMD_HGRN2_CHUNK_FROM", "256"))  # longest run from which a step is chunked
# tokens per chunk. Measured on a 2048-token prompt (32 heads x 64 x 64): 32 / 64 / 128 tokens give 0.66 / 0.62 /
# 0.63 ms per layer against 1.22 ms token by token
HGRN2_CHUNK_LEN = int(os.environ.get("LLMD_HGRN2_CHUNK_LEN", "64"))


def hgrn2_scan(p, H: int, dk: int, dv: int, f_bias, lower, norm_w, eps: float, state, seq):
    """HGRN2 over a step's runs. ``p`` [T, >= 2 H dk + H dv] = [q | f | v] as projected. Per token and
    head, all fp32: q <- silu(q); f <- lower + (1 - lower) sigmoid(f + f_bias) (both fp32 [H dk]); then

        S <- diag(f) S + (1 - f) v^T;  o = S^T q

    (f scales the rows of S) and o / rms(o) * norm_w [dv]. ``state`` [slots, H, dk, dv] fp32 is
    continued (seq_init) and written back. Returns [T, H dv].

    A step with a long run (a prompt) takes the chunked form: the recurrence is linear in S, so the runs
    are cut into chunks (``SeqMeta.scan_chunks``) that are scanned side by side - once from zero for
    each chunk's own contribution, then, after the chunks' start states have been linked in order, once
    more with the read-outs. Steps of short runs go token by token."""
    out = torch.empty(p.shape[0], H * dv, dtype=p.dtype, device=p.device)
    if not p.is_cuda:
        return ref.hgrn2_scan(p, H, dk, dv, f_bias, lower, norm_w, eps, state, seq.seq_start, seq.seq_slot,
                              seq.seq_init, out)
    chunks, nc = None, 0
    if HGRN2_CHUNKED and seq.max_q >= HGRN2_CHUNK_FROM and seq.q_lens is not None:
        chunks, nc = seq.scan_chunks(HGRN2_CHUNK_LEN)
    native().hgrn2_scan(p, int(H), int(dk), int(dv), f_bias, lower, norm_w, float(eps), state, seq.seq_start,
                        seq.seq_slot, seq.seq_init, out, chunks, nc)
    return out
