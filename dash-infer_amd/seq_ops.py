"""Tensor-level wrappers over libdashinfer_hip_seq.so (torch: device memory and streams only).

Activations between operators are f32 tensors, possibly column slices of a wider buffer (row stride = stride(0)); weights
stay in the type the checkpoint stores (bf16 or f32: both widen to f32 exactly).  `math` selects how dihip_linear
multiplies: seq_capi.MATH_F32 (every product and sum in f32) or MATH_BF16 (bf16 operands, f32 accumulation).
"""
import ctypes as C

import torch

from . import seq_capi
from .seq_capi import ACT, MATH_BF16, MATH_F32, MATH_F32_STREAM, check, lib

_DT = {torch.float32: seq_capi.F32, torch.bfloat16: seq_capi.BF16}
F32_CODE = seq_capi.F32


def dt(t):
    return _DT[t.dtype]


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _rows(t):
    assert t.dim() == 2 and t.stride(1) == 1, "row-major rows (a column slice of a wider buffer is fine)"
    return t.stride(0)


def linear(x, w, bias=None, out=None, act=None, act_cols=None, mul=None, math=MATH_F32, groups=1, x_groups=None):
    """y = epilogue(x . w^T + bias).  w: [N, K] (groups == 1) or [groups, N, K]; x: [T, x_groups * K] (group g reads the K
    columns from (g % x_groups) * K); y: [T, groups * N].  act on the output columns act_cols = (lo, hi) (default: all);
    mul: f32 [T, groups * N] multiplied on the output."""
    if w.dim() == 2:
        N, K = w.shape
    else:
        assert w.shape[0] == groups
        _, N, K = w.shape
    xg = groups if x_groups is None else x_groups
    T = x.shape[0]
    assert x.shape[1] == xg * K and w.is_contiguous() and (bias is None or (bias.is_contiguous() and bias.dtype == w.dtype))
    y = out if out is not None else torch.empty(T, groups * N, dtype=torch.float32, device=x.device)
    assert y.shape == (T, groups * N)
    lo, hi = (0, groups * N) if act_cols is None else act_cols
    if act is None:
        lo = hi = 0
    check(lib().dihip_linear(stream(), ptr(x), dt(x), _rows(x), K, xg, ptr(w), dt(w), ptr(bias), ptr(y), dt(y), _rows(y), N,
                             ptr(mul), _rows(mul) if mul is not None else 0, T, N, K, groups, ACT[act], lo, hi, math), "dihip_linear")
    return y


def embed_sum(ids, table, rows2=None, table2=None, out=None):
    T, K = ids.shape[0], table.shape[1]
    h = out if out is not None else torch.empty(T, K, dtype=torch.float32, device=table.device)
    assert table2 is None or (table2.dtype == table.dtype and table2.shape[1] == K)
    check(lib().dihip_embed_sum(stream(), ptr(h), ptr(ids), ptr(table), ptr(rows2), ptr(table2), dt(table), T, K), "dihip_embed_sum")
    return h


def embed_rows(ids, table, col0=0, cols=None, scale=1.0, out=None):
    """out[t] = table[ids[t], col0 : col0 + cols] * scale; out: rows of any stride, f32 or bf16 (default: a new f32 tensor)"""
    T = ids.shape[0]
    K = table.shape[1] - col0 if cols is None else cols
    y = out if out is not None else torch.empty(T, K, dtype=torch.float32, device=table.device)
    assert y.shape == (T, K) and table.is_contiguous()
    check(lib().dihip_embed_rows(stream(), ptr(y), dt(y), _rows(y), ptr(ids), ptr(table), dt(table), table.shape[1], int(col0), float(scale),
                                 T, K), "dihip_embed_rows")
    return y


def rmsnorm(x, gamma, eps, row_idx=None, out=None, gamma_add=0.0, out_scale=1.0):
    """y = x / rms(x) * (gamma_add + gamma) * out_scale"""
    M = x.shape[0] if row_idx is None else row_idx.shape[0]
    K = gamma.shape[0]
    assert x.shape[1] == K and x.dtype == torch.float32
    y = out if out is not None else torch.empty(M, K, dtype=torch.float32, device=x.device)
    check(lib().dihip_rmsnorm_strided(stream(), ptr(y), dt(y), _rows(y), ptr(x), _rows(x), ptr(row_idx), ptr(gamma), dt(gamma), float(gamma_add),
                                      float(out_scale), float(eps), M, K), "dihip_rmsnorm_strided")
    return y


def residual_norm_step(x_in, eps, m=None, gamma_m=None, add_m=0.0, x_out=None, gamma_h=None, add_h=0.0, h=None, copy=None):
    """x_out = x_in + m / rms(m) * (add_m + gamma_m) (m None: x_in itself); copy <- x_out (rows of any stride, f32 or bf16);
    h <- x_out / rms(x_out) * (add_h + gamma_h) (f32 or bf16).  -> x_out"""
    T, K = x_in.shape
    assert x_in.is_contiguous() and x_in.dtype == torch.float32
    if m is not None:
        x_out = x_in if x_out is None else x_out
        assert x_out.is_contiguous() and x_out.shape == (T, K) and m.shape == (T, K) and m.dtype == torch.float32 and gamma_m.shape[0] == K
    assert h is None or (h.shape == (T, K) and gamma_h.shape[0] == K)
    assert copy is None or copy.shape == (T, K)
    g = gamma_m if gamma_m is not None else gamma_h
    assert gamma_m is None or gamma_h is None or gamma_m.dtype == gamma_h.dtype
    check(lib().dihip_residual_norm_step(stream(), ptr(x_out), ptr(x_in), ptr(m), _rows(m) if m is not None else 0, ptr(gamma_m), float(add_m),
                                         ptr(gamma_h), float(add_h), dt(g) if g is not None else F32_CODE, float(eps), ptr(copy),
                                         dt(copy) if copy is not None else F32_CODE, _rows(copy) if copy is not None else 0, ptr(h),
                                         dt(h) if h is not None else F32_CODE, _rows(h) if h is not None else 0, T, K), "dihip_residual_norm_step")
    return x_out if m is not None else x_in


def norm_span_append(table, x, gamma, eps, tok_slot, tok_pos):
    """table: a SpanTable (seq_state) of rows of x.shape[1] elements"""
    T, K = x.shape
    assert K == table.row_elems and x.dtype == torch.float32
    check(lib().dihip_norm_span_append(stream(), ptr(table.ptrs), table.max_spans, table.span_len, _DT[table.dtype], ptr(x), _rows(x),
                                       ptr(gamma), dt(gamma), float(eps), ptr(tok_slot), ptr(tok_pos), T, K), "dihip_norm_span_append")


def norm_residual_mix(x_in, m, gamma, eps, x_out, stack=None, mix_w=None, n_mix=0, x_mix=None, next16=None):
    """next16: optional bf16 [T, K] copy of what the next product reads (x_mix where n_mix > 0, else x_out)"""
    T, K = x_in.shape
    assert x_in.is_contiguous() and x_out.is_contiguous() and m.shape == (T, K)
    assert next16 is None or (next16.dtype == torch.bfloat16 and next16.is_contiguous() and next16.shape == (T, K))
    if n_mix:
        assert stack.is_contiguous() and stack.shape[0] >= n_mix and x_mix.is_contiguous() and mix_w.shape[0] >= n_mix
    check(lib().dihip_norm_residual_mix(stream(), ptr(x_out), ptr(x_in), ptr(m), _rows(m), ptr(gamma), dt(gamma), float(eps),
                                        ptr(stack), stack.stride(0) if n_mix else 0, ptr(mix_w), n_mix, ptr(x_mix), ptr(next16), T, K),
          "dihip_norm_residual_mix")
    return x_out


def latent_window_attn(q, table, sink, tok_slot, tok_pos, H, window, scale, math=MATH_F32, out=None):
    T = q.shape[0]
    R = table.row_elems
    assert q.shape[1] == H * R and q.dtype == torch.float32
    o = out if out is not None else torch.empty(T, H * R, dtype=torch.float32, device=q.device)
    check(lib().dihip_latent_window_attn(stream(), ptr(o), _rows(o), ptr(q), _rows(q), ptr(table.ptrs), table.max_spans, table.span_len,
                                         _DT[table.dtype], ptr(sink), dt(sink) if sink is not None else 0, ptr(tok_slot), ptr(tok_pos),
                                         T, H, R, int(window), float(scale), math), "dihip_latent_window_attn")
    return o


def latent_attn_mc_supported(table):
    return bool(lib().dihip_latent_window_attn_mc_supported(table.row_elems, table.span_len, _DT[table.dtype]))


def latent_window_attn_mc(q, table, sink, tok_pos, ent_slot, ent_row0, ent_count, max_count, max_pos, H, window, scale, out=None, nsplit=None):
    """the matrix-core form (bf16 cache): rows as portions; max_count / max_pos: the largest portion and position of the step
    (host numbers: they size the grid and the split of the key walk)"""
    T, R, E = q.shape[0], table.row_elems, ent_slot.shape[0]
    o = out if out is not None else torch.empty(T, H * R, dtype=torch.float32, device=q.device)
    if nsplit is None:       # fill the chip: ~2 workgroups per CU; at least 2 key tiles (64 keys) per workgroup
        blocks = max(1, E * ((max_count * H + 63) // 64))
        keys = min(max_pos + 1, window) if window > 0 else max_pos + 1
        nsplit = max(1, min(512 // blocks, (keys + 63) // 64))
    ws = None
    if nsplit > 1:
        ws = torch.empty(int(lib().dihip_latent_window_attn_mc_workspace_bytes(T, H, R, nsplit)), dtype=torch.uint8, device=q.device)
    check(lib().dihip_latent_window_attn_mc(stream(), ptr(o), _rows(o), ptr(q), _rows(q), ptr(table.ptrs), table.max_spans, table.span_len,
                                            ptr(sink), dt(sink) if sink is not None else 0, ptr(tok_pos), ptr(ent_slot), ptr(ent_row0),
                                            ptr(ent_count), E, int(max_count), T, H, R, int(window), float(scale), int(nsplit), ptr(ws),
                                            ws.numel() if ws is not None else 0), "dihip_latent_window_attn_mc")
    return o


def causal_conv_state(x, w, bias, tail, tok_slot, tok_off, out=None, act=None):
    """act: None or "silu" on the result"""
    T, Cn = x.shape
    taps = w.shape[1]
    u = out if out is not None else torch.empty(T, Cn, dtype=torch.float32, device=x.device)
    check(lib().dihip_causal_conv_state(stream(), ptr(u), _rows(u), ptr(x), _rows(x), ptr(w), ptr(bias), dt(w), ptr(tail), ptr(tok_slot),
                                        ptr(tok_off), T, Cn, taps, ACT[act]), "dihip_causal_conv_state")
    return u


def conv_tail_update(tail, x, taps, ent_slot, ent_row0, ent_count):
    check(lib().dihip_conv_tail_update(stream(), ptr(tail), ptr(x), _rows(x), ptr(ent_slot), ptr(ent_row0), ptr(ent_count),
                                       ent_slot.shape[0], x.shape[1], taps), "dihip_conv_tail_update")


CHUNKED_RECURRENCE_ROWS = 256   # portions from this length on run as chunks side by side


def gated_recurrence(r, i, u, y, lam, decay, state, ent_slot, ent_row0, ent_count, out=None, max_count=None):
    """max_count: the step's largest portion (a host number); given and >= CHUNKED_RECURRENCE_ROWS: the chunk-parallel form"""
    T, Cn = u.shape
    assert _rows(r) == _rows(i)
    o = out if out is not None else torch.empty(T, Cn, dtype=torch.float32, device=u.device)
    if max_count is not None and max_count >= CHUNKED_RECURRENCE_ROWS:
        E = ent_slot.shape[0]
        ws = torch.empty(int(lib().dihip_gated_recurrence_chunked_workspace_bytes(E, max_count, Cn)), dtype=torch.uint8, device=u.device)
        check(lib().dihip_gated_recurrence_chunked(stream(), ptr(o), _rows(o), ptr(r), ptr(i), _rows(r), ptr(u), _rows(u), ptr(y), _rows(y),
                                                   ptr(lam), dt(lam), float(decay), ptr(state), ptr(ent_slot), ptr(ent_row0), ptr(ent_count),
                                                   E, int(max_count), Cn, ptr(ws), ws.numel()), "dihip_gated_recurrence_chunked")
        return o
    check(lib().dihip_gated_recurrence(stream(), ptr(o), _rows(o), ptr(r), ptr(i), _rows(r), ptr(u), _rows(u), ptr(y), _rows(y), ptr(lam),
                                       dt(lam), float(decay), ptr(state), ptr(ent_slot), ptr(ent_row0), ptr(ent_count),
                                       ent_slot.shape[0], Cn), "dihip_gated_recurrence")
    return o


def linear_segmented(x, w, seg, row_map, seg_max_rows, R, bias=None, out=None, act=None, math=MATH_F32):
    """rows grouped by owner: w [groups, N, K]; output row r (seg[g] <= r < seg[g + 1]) = x[row_map[r]] . w[g]^T (+ bias[g]);
    seg_max_rows: a host-known bound on one group's rows -> [R, N] f32"""
    groups, N, K = w.shape
    assert x.shape[1] == K and w.is_contiguous() and seg.dtype == torch.int32 and seg.shape[0] >= groups + 1
    y = out if out is not None else torch.empty(R, N, dtype=torch.float32, device=x.device)
    assert y.shape == (R, N)
    check(lib().dihip_linear_segmented(stream(), ptr(x), dt(x), _rows(x), ptr(w), dt(w), ptr(bias), ptr(y), dt(y), _rows(y), R, N, K, groups,
                                       ptr(seg), ptr(row_map), int(seg_max_rows), ACT[act], math), "dihip_linear_segmented")
    return y


def add_dyt(x_in, a=None, b=None, norm=None, x_out=None, row_idx=None, want16=False):
    """x_out = x_in + (a + b);  h = tanh(alpha * x_out) * w + bias for norm = (alpha, w, bias) -> (h f32, h16 bf16 or None)"""
    K = x_in.shape[1]
    M = x_in.shape[0] if row_idx is None else row_idx.shape[0]
    assert x_in.is_contiguous() and x_in.dtype == torch.float32 and (x_out is None or x_out.is_contiguous())
    h = h16 = None
    alpha, w, bias = 0.0, None, None
    if norm is not None:
        alpha, w, bias = norm
        if want16:
            h16 = torch.empty(M, K, dtype=torch.bfloat16, device=x_in.device)
        else:
            h = torch.empty(M, K, dtype=torch.float32, device=x_in.device)
    check(lib().dihip_add_dyt(stream(), ptr(x_out), ptr(x_in), ptr(a), _rows(a) if a is not None else 0, ptr(b), _rows(b) if b is not None else 0,
                              ptr(row_idx), float(alpha), ptr(w), ptr(bias), dt(w) if w is not None else F32_CODE, ptr(h), ptr(h16), M, K),
          "dihip_add_dyt")
    return h, h16


def qkv_prep_append(a, q_off, k_off, v_off, H, G, D, DV, qnorm, knorm, eps, freq, rot_dims, layout, mag, lam, vfirst_in, vfirst_out,
                    ktable, vtable, tok_slot, tok_pos, maps=1):
    """norm + rotation of the q / k columns of the rows a (q in place), value mixing, append of k and v to their pages; maps: query
    vectors per head and key vectors per key head"""
    T = a.shape[0]
    assert a.dtype == torch.float32 and ktable.row_elems == G * maps * D and vtable.row_elems == G * DV and ktable.dtype == vtable.dtype
    vf = vfirst_in if vfirst_in is not None else vfirst_out
    wn = qnorm if qnorm is not None else knorm
    check(lib().dihip_qkv_prep_append(stream(), ptr(a), _rows(a), q_off, k_off, v_off, H, G, D, DV, int(maps), ptr(qnorm), ptr(knorm),
                                      dt(wn) if wn is not None else F32_CODE, float(eps), ptr(freq), int(rot_dims), int(layout), float(mag),
                                      float(lam), ptr(vfirst_in), ptr(vfirst_out), _rows(vf) if vf is not None else 0, ptr(ktable.ptrs),
                                      ptr(vtable.ptrs), ktable.max_spans, ktable.span_len, _DT[ktable.dtype], ptr(tok_slot), ptr(tok_pos), T),
          "dihip_qkv_prep_append")


SINK_NONE, SINK_PER_HEAD, SINK_ZERO = 0, 1, 2


def gqa_attn(q, ktable, vtable, tok_slot, tok_pos, H, G, D, DV, scale, sink=None, sink_mode=SINK_NONE, softcap=0.0, gate=None, out=None,
             maps=1, window=0, keep_first=0):
    """q: f32 [T, >= H * maps * D] rows (a column slice is fine); gate: f32 [T, >= H] or None -> f32 [T, H * maps * DV].  window > 0:
    a row reads the keys less than `window` positions back and the first keep_first keys of its sequence"""
    T = q.shape[0]
    o = out if out is not None else torch.empty(T, H * maps * DV, dtype=torch.float32, device=q.device)
    check(lib().dihip_gqa_attn(stream(), ptr(o), _rows(o), ptr(q), _rows(q), ptr(ktable.ptrs), ptr(vtable.ptrs), ktable.max_spans, ktable.span_len,
                               _DT[ktable.dtype], ptr(sink), dt(sink) if sink is not None else F32_CODE, int(sink_mode), float(softcap or 0.0),
                               ptr(gate), _rows(gate) if gate is not None else 0, ptr(tok_slot), ptr(tok_pos), T, H, G, D, DV, float(scale),
                               int(maps), int(window or 0), int(keep_first or 0)), "dihip_gqa_attn")
    return o


def gqa_attn_mc_supported(D, DV, table):
    """head sizes D / DV on pages like those of `table`"""
    return bool(lib().dihip_gqa_attn_mc_supported(int(D), int(DV), table.span_len, _DT[table.dtype]))


def gqa_attn_mc(q, ktable, vtable, tok_pos, ent_slot, ent_row0, ent_count, max_count, max_pos, H, G, D, DV, scale, sink=None,
                sink_mode=SINK_NONE, softcap=0.0, gate=None, out=None, nsplit=None, maps=1, window=0, keep_first=0, diff=None):
    """the matrix-core form (bf16 pages); max_count / max_pos: the largest portion and position of the step (host numbers).
    diff = (lam, out_scale, eps, y): with two maps, y [T, H * DV] <- maps_diff_norm of the result (inside the merge of a split walk)
    and y is returned"""
    T, E = q.shape[0], ent_slot.shape[0]
    window, keep_first = int(window or 0), int(keep_first or 0)
    o = out if out is not None else torch.empty(T, H * maps * DV, dtype=torch.float32, device=q.device)
    if nsplit is None:       # fill the chip: ~2 workgroups per CU; at least 2 key tiles (64 keys) per workgroup
        blocks = max(1, E * G * maps * ((max_count * (H // G) + 63) // 64))
        keys = min(max_pos + 1, window + keep_first) if window > 0 else max_pos + 1
        nsplit = max(1, min(512 // blocks, (keys + 63) // 64))
    ws = None
    if nsplit > 1:
        ws = torch.empty(int(lib().dihip_gqa_attn_mc_workspace_bytes(T, H * maps, DV, nsplit)), dtype=torch.uint8, device=q.device)
    check(lib().dihip_gqa_attn_mc(stream(), ptr(o), _rows(o), ptr(q), _rows(q), ptr(ktable.ptrs), ptr(vtable.ptrs), ktable.max_spans,
                                  ktable.span_len, ptr(sink), dt(sink) if sink is not None else F32_CODE, int(sink_mode), float(softcap or 0.0),
                                  ptr(gate), _rows(gate) if gate is not None else 0, ptr(tok_pos), ptr(ent_slot), ptr(ent_row0), ptr(ent_count),
                                  E, int(max_count), T, H, G, D, DV, float(scale), int(maps), window, keep_first, int(nsplit), ptr(ws),
                                  ws.numel() if ws is not None else 0, ptr(diff[3]) if diff else None, dt(diff[3]) if diff else F32_CODE,
                                  _rows(diff[3]) if diff else 0, float(diff[0]) if diff else 0.0, float(diff[1]) if diff else 0.0,
                                  float(diff[2]) if diff else 0.0), "dihip_gqa_attn_mc")
    return diff[3] if diff else o


def maps_diff_norm(x, lam, out_scale, eps, H, DV, out=None):
    """x: f32 [T, H * 2 * DV] (two maps per head side by side) -> (first - lam * second) / its root mean square * out_scale, [T, H * DV]"""
    T = x.shape[0]
    y = out if out is not None else torch.empty(T, H * DV, dtype=torch.float32, device=x.device)
    check(lib().dihip_maps_diff_norm(stream(), ptr(y), dt(y), _rows(y), ptr(x), _rows(x), float(lam), float(out_scale), float(eps), T, H, DV),
          "dihip_maps_diff_norm")
    return y


CHUNKED_GLA_ROWS = 128   # portions from this length on run as chunks side by side


def gla(q, k, v, z, q_scale, tau, state, ent_slot, ent_row0, ent_count, max_count, H, D, DV, out=None, chunked=None):
    """q, k, z: f32 [T, >= H * D] rows, v: [T, >= H * DV]; state [slots, H, D, DV] f32 -> f32 [T, H * DV]"""
    T, E = q.shape[0], ent_slot.shape[0]
    assert state.shape[1:] == (H, D, DV) and state.is_contiguous()
    o = out if out is not None else torch.empty(T, H * DV, dtype=torch.float32, device=q.device)
    if chunked is None:
        chunked = max_count >= CHUNKED_GLA_ROWS
    chunked = 1 if chunked else 0
    ws = torch.empty(int(lib().dihip_gla_workspace_bytes(T, E, int(max_count), H, D, DV, chunked)), dtype=torch.uint8, device=q.device)
    check(lib().dihip_gla(stream(), ptr(o), _rows(o), ptr(q), _rows(q), ptr(k), _rows(k), ptr(v), _rows(v), ptr(z), _rows(z), float(q_scale),
                          float(tau), ptr(state), ptr(ent_slot), ptr(ent_row0), ptr(ent_count), T, E, int(max_count), H, D, DV, chunked,
                          ptr(ws), ws.numel()), "dihip_gla")
    return o


def head_rmsnorm_mul(x, gamma, eps, H, DV, mul=None, out=None):
    T = x.shape[0]
    y = out if out is not None else torch.empty(T, H * DV, dtype=torch.float32, device=x.device)
    check(lib().dihip_head_rmsnorm_mul(stream(), ptr(y), dt(y), _rows(y), ptr(x), _rows(x), ptr(gamma), dt(gamma), float(eps), ptr(mul),
                                       _rows(mul) if mul is not None else 0, T, H, DV), "dihip_head_rmsnorm_mul")
    return y


ROUTE_CHOSEN_SOFTMAX, ROUTE_SCORES = 0, 1      # weights = softmax over the chosen logits / the chosen softmax scores over their sum
UNIT_CLAMPED, UNIT_SILU = 0, 1


def moe_route(logits, top, scoring=ROUTE_CHOSEN_SOFTMAX, correction=None, groups=(1, 1)):
    """groups = (count, keep): only experts of the `keep` best of `count` equal groups of neighbours can be chosen
    -> ids [T, top] i32, wts [T, top] f32, seg [E + 1], src_row [T * top], dst [T * top]"""
    T, E = logits.shape
    dev = logits.device
    ints = torch.empty(T * top * 3 + 2 * E + 1, dtype=torch.int32, device=dev)
    ids, src_row, dst = ints[: T * top], ints[T * top: 2 * T * top], ints[2 * T * top: 3 * T * top]
    counts, seg = ints[3 * T * top: 3 * T * top + E], ints[3 * T * top + E:]
    wts = torch.empty(T, top, dtype=torch.float32, device=dev)
    assert correction is None or (correction.shape == (E,) and correction.is_contiguous())
    check(lib().dihip_seq_moe_route(stream(), ptr(logits), _rows(logits), ptr(ids), ptr(wts), ptr(counts), ptr(seg), ptr(src_row), ptr(dst),
                                    T, E, int(top), int(scoring), ptr(correction), dt(correction) if correction is not None else F32_CODE,
                                    int(groups[0]), int(groups[1])), "dihip_seq_moe_route")
    return ids.view(T, top), wts, seg, src_row, dst


def moe_glu(gu, F, limit, slope, out, unit=UNIT_CLAMPED):
    R = gu.shape[0]
    check(lib().dihip_seq_moe_glu(stream(), ptr(out), dt(out), _rows(out), ptr(gu), _rows(gu), R, F, float(limit), float(slope), int(unit)),
          "dihip_seq_moe_glu")
    return out


def moe_combine(rows, dst, wts, T, top, out=None, ids=None, n_real=0, own=None, add=None):
    """ids / n_real / own: choices >= n_real are identity experts, their row is own[t] (f32 or bf16); add: f32 rows added per token"""
    K = rows.shape[1]
    o = out if out is not None else torch.empty(T, K, dtype=torch.float32, device=rows.device)
    check(lib().dihip_seq_moe_combine(stream(), ptr(o), _rows(o), ptr(rows), _rows(rows), ptr(dst), ptr(wts), T, int(top), K, ptr(ids), int(n_real),
                                      ptr(own), dt(own) if own is not None else F32_CODE, _rows(own) if own is not None else 0, ptr(add),
                                      _rows(add) if add is not None else 0), "dihip_seq_moe_combine")
    return o


def residual_layernorm(x_in, w=None, a=None, b=None, mult=1.0, eps=1e-5, x_out=None, row_idx=None, bias=None, out_dtype=torch.float32):
    """x_out = x_in + mult * (a + b);  h = layer_norm(x_out) * w (+ bias)  (mean and variance over the row) -> h (None without w).
    row_idx: the norm of the chosen rows of x_in alone."""
    K = x_in.shape[1]
    M = x_in.shape[0] if row_idx is None else row_idx.shape[0]
    assert x_in.is_contiguous() and x_in.dtype == torch.float32 and (x_out is None or x_out.is_contiguous())
    assert a is None or x_out is not None
    h = torch.empty(M, K, dtype=out_dtype, device=x_in.device) if w is not None else None
    check(lib().dihip_residual_layernorm(stream(), ptr(x_out), ptr(x_in), ptr(a), _rows(a) if a is not None else 0, ptr(b),
                                         _rows(b) if b is not None else 0, float(mult), ptr(row_idx), ptr(w), ptr(bias),
                                         dt(w) if w is not None else F32_CODE, float(eps), ptr(h), dt(h) if h is not None else F32_CODE,
                                         _rows(h) if h is not None else 0, M, K), "dihip_residual_layernorm")
    return h


def polynorm(z, coef, eps, out):
    """out = c0 z / rms(z) + c1 z^2 / rms(z^2) + c2 z^3 / rms(z^3) + c3 over the rows of z (f32); coef: the four numbers"""
    T, F = z.shape
    assert z.dtype == torch.float32 and out.shape == (T, F) and coef.numel() == 4 and coef.is_contiguous()
    check(lib().dihip_polynorm(stream(), ptr(out), dt(out), _rows(out), ptr(z), _rows(z), ptr(coef), dt(coef), float(eps), T, F), "dihip_polynorm")
    return out


def rmsnorm_pair(xa, wa, xb, wb, coef, eps, out=None):
    """coef * (xa / rms(xa) * wa + xb / rms(xb) * wb) -> f32 [T, K]"""
    T, K = xa.shape
    assert xb.shape == (T, K) and xa.dtype == xb.dtype == torch.float32 and wa.dtype == wb.dtype and wa.shape[0] == wb.shape[0] == K
    y = out if out is not None else torch.empty(T, K, dtype=torch.float32, device=xa.device)
    check(lib().dihip_rmsnorm_pair(stream(), ptr(y), _rows(y), ptr(xa), _rows(xa), ptr(wa), ptr(xb), _rows(xb), ptr(wb), dt(wa), float(coef),
                                   float(eps), T, K), "dihip_rmsnorm_pair")
    return y


def gate_group_rmsnorm(o, z, w, eps, heads, P, groups, x=None, skip=None, out=None):
    """v = (o + skip[head] * x) * silu(z); out = v / rms(v over each of `groups` equal parts of the row) * w"""
    T = o.shape[0]
    y = out if out is not None else torch.empty(T, heads * P, dtype=torch.float32, device=o.device)
    assert o.dtype == z.dtype == torch.float32 and w.shape[0] == heads * P and (skip is None or (skip.dtype == w.dtype and x is not None))
    check(lib().dihip_gate_group_rmsnorm(stream(), ptr(y), dt(y), _rows(y), ptr(o), _rows(o), ptr(x), _rows(x) if x is not None else 0,
                                         ptr(skip), ptr(z), _rows(z), ptr(w), dt(w), float(eps), T, int(heads), int(P), int(groups)),
          "dihip_gate_group_rmsnorm")
    return y


def latent_rope_append(table, ckv, gamma, eps, R, rot, freq, q_rot, ql, H, tok_slot, tok_pos, append=True):
    """table: the SpanTable of rows [R latent | rot key part | padding]; append False: only the queries' rotated parts are written
    (a layer that reads another layer's pages)"""
    T, Rp = ql.shape[0], table.row_elems
    assert ql.dtype == q_rot.dtype == torch.float32 and ql.shape[1] == H * Rp and q_rot.shape[1] == H * rot
    assert not append or (ckv.dtype == torch.float32 and ckv.shape[1] == R + rot)
    check(lib().dihip_latent_rope_append(stream(), ptr(table.ptrs) if append else None, table.max_spans, table.span_len, _DT[table.dtype],
                                         ptr(ckv) if append else None, _rows(ckv) if append else 0, ptr(gamma) if append else None,
                                         dt(gamma) if append and gamma is not None else F32_CODE, float(eps), int(R), int(rot), int(Rp),
                                         ptr(freq), ptr(q_rot), _rows(q_rot), ptr(ql), _rows(ql), int(H), ptr(tok_slot), ptr(tok_pos), T),
          "dihip_latent_rope_append")


def ssd(x, B, Cq, dtr, dt_bias, a_log, state, ent_slot, ent_row0, ent_count, max_count, H, G, D, DV, out=None, chunked=None):
    """state-space scan with a scalar decay per head: x [T, >= H * DV], B / Cq [T, >= G * D], dtr [T, >= H] f32 rows; state
    [slots, H, D, DV] f32 -> f32 [T, H * DV]"""
    T, E = x.shape[0], ent_slot.shape[0]
    assert state.shape[1:] == (H, D, DV) and state.is_contiguous() and dt_bias.dtype == a_log.dtype
    o = out if out is not None else torch.empty(T, H * DV, dtype=torch.float32, device=x.device)
    if chunked is None:
        chunked = max_count >= CHUNKED_GLA_ROWS
    chunked = 1 if chunked else 0
    ws = torch.empty(int(lib().dihip_gla_workspace_bytes(T, E, int(max_count), H, D, DV, chunked)), dtype=torch.uint8, device=x.device)
    check(lib().dihip_ssd(stream(), ptr(o), _rows(o), ptr(x), _rows(x), ptr(B), _rows(B), ptr(Cq), _rows(Cq), ptr(dtr), _rows(dtr), ptr(dt_bias),
                          ptr(a_log), dt(a_log), ptr(state), ptr(ent_slot), ptr(ent_row0), ptr(ent_count), T, E, int(max_count), int(H), int(G),
                          int(D), int(DV), chunked, ptr(ws), ws.numel()), "dihip_ssd")
    return o


TALK_MAX_HEADS = 64
TALK_FEW_ROWS = 64      # steps of at most this many rows spread the attention with mixed maps over (row, head, chunk) workgroups


def talk_attn(q, ktable, vtable, tok_slot, tok_pos, max_pos, H, G, D, DV, scale, talk, temp=None, gate=None, window=0, out=None, nsplit=None):
    """attention whose softmax maps are mixed between the heads (talk [H, H]) after the softmax; temp [H]: a multiplier per head on
    the scores; gate: f32 [T, >= H * DV] multiplier.  max_pos: the step's last position (a host number: it sizes the split of the
    key walk for few rows) -> [T, H * DV] (f32, or `out`)"""
    T = q.shape[0]
    window = int(window or 0)
    o = out if out is not None else torch.empty(T, H * DV, dtype=torch.float32, device=q.device)
    assert talk.shape == (H, H) and talk.is_contiguous() and (temp is None or (temp.dtype == talk.dtype and temp.shape == (H,)))
    keys = min(max_pos + 1, window) if window > 0 else max_pos + 1
    if nsplit is None and T <= TALK_FEW_ROWS:      # few rows (decoding): the work spread over rows, heads and chunks
        ws = torch.empty(int(lib().dihip_talk_attn_few_workspace_bytes(T, H, DV, keys)), dtype=torch.uint8, device=q.device)
        check(lib().dihip_talk_attn_few(stream(), ptr(o), dt(o), _rows(o), ptr(q), _rows(q), ptr(ktable.ptrs), ptr(vtable.ptrs), ktable.max_spans,
                                        ktable.span_len, _DT[ktable.dtype], ptr(temp), ptr(talk), dt(talk), ptr(gate),
                                        _rows(gate) if gate is not None else 0, ptr(tok_slot), ptr(tok_pos), T, H, G, D, DV, float(scale), window,
                                        int(keys), ptr(ws), ws.numel()), "dihip_talk_attn_few")
        return o
    if nsplit is None:       # one workgroup per (row, part of the walk)
        nsplit = max(1, min(256 // max(T, 1), (keys + 63) // 64))
    ws = torch.empty(int(lib().dihip_talk_attn_workspace_bytes(T, H, DV, nsplit)), dtype=torch.uint8, device=q.device)
    check(lib().dihip_talk_attn(stream(), ptr(o), dt(o), _rows(o), ptr(q), _rows(q), ptr(ktable.ptrs), ptr(vtable.ptrs), ktable.max_spans,
                                ktable.span_len, _DT[ktable.dtype], ptr(temp), ptr(talk), dt(talk), ptr(gate),
                                _rows(gate) if gate is not None else 0, ptr(tok_slot), ptr(tok_pos), T, H, G, D, DV, float(scale), window,
                                int(nsplit), ptr(ws), ws.numel()), "dihip_talk_attn")
    return o


TALK_MC_MIN_ROWS = 16    # steps whose largest portion has fewer rows (decoding) take the split row kernel


def talk_attn_mc_supported(H, G, D, DV, table):
    return bool(lib().dihip_talk_attn_mc_supported(int(H), int(G), int(D), int(DV), table.span_len, _DT[table.dtype]))


def talk_attn_mc(q, ktable, vtable, tok_pos, ent_slot, ent_row0, ent_count, max_count, H, G, D, DV, scale, talk32, temp=None, gate=None, window=0,
                 out=None):
    """the matrix-core form of talk_attn (bf16 pages): rows as portions; talk32: the mixing matrix as f32 [H, H]"""
    T, E = q.shape[0], ent_slot.shape[0]
    o = out if out is not None else torch.empty(T, H * DV, dtype=torch.float32, device=q.device)
    ws = torch.empty(int(lib().dihip_talk_attn_mc_workspace_bytes(T, H)), dtype=torch.uint8, device=q.device)
    assert talk32.dtype == torch.float32 and talk32.shape == (H, H) and talk32.is_contiguous() and q.dtype == torch.float32
    check(lib().dihip_talk_attn_mc(stream(), ptr(o), dt(o), _rows(o), ptr(q), _rows(q), ptr(ktable.ptrs), ptr(vtable.ptrs), ktable.max_spans,
                                   ktable.span_len, ptr(temp), dt(temp) if temp is not None else F32_CODE, ptr(talk32), ptr(gate),
                                   _rows(gate) if gate is not None else 0, ptr(tok_pos), ptr(ent_slot), ptr(ent_row0), ptr(ent_count), E,
                                   int(max_count), T, H, G, D, DV, float(scale), int(window or 0), ptr(ws), ws.numel()), "dihip_talk_attn_mc")
    return o
