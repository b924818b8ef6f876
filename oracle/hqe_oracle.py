"""CPU oracle for the quantized-KV decode-attention path.  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU and with plain torch tensor ops, what the reference
computes on its GPU path.  It is imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py`` -- never by the product package.

Every function cites the reference lines it follows (paths relative to the reference
checkout).  How each function is pinned (known answers, closed forms, brute force) is
listed next to it; the checks themselves live in ``tests/test_oracle.py`` and
``tests/golden/``.

Pinned:
  pack_along_last_dim / unpack_along_last_dim   closed form, round trip, KAT 0xE4E4E4E4
  uniform_group_quantize_pack_last_dim          arange(128) known answer, 8-bit identity,
                                                invariants (min->0, 0<=c<=qmax, |x-dq|<=s/2)
  uniform_group_dequantize_unpack_last_dim      closed form on hand-computed values
  gemv_uniform_group                            special cases that collapse to integer
                                                mat-vec / torch.matmul
  qkv_matmul                                    permutation invariance against dense attention
  compress_cache / rerank_after_eviction        brute force against a per-block history model and Python sets
  1-bit uniform class (bit == 1 above)          arange known answer (scale 31, words 0xFFFF0000), tie -> even code
  normal_group_(de)quantize (1-bit table)       arange(32) known answer worked out with numpy float16, unbiased
                                                std / mean against float64, code == sign of x - mean
  DecodeLayerOracle / ImportanceRing            bookkeeping invariants over a prompt and 40 decode steps (every
                                                token in one class, the residual or evicted; class sizes follow
                                                the ratio schedule; two blocks stay fp16)
  KiviLayerOracle                               closed-form lengths after every step (whole blocks of K, all
                                                but the last R tokens of V quantised) and equality of its decode
                                                step with plain attention over the reconstructed cache

Parity unpinned (no reference fixture exists and only a run of the original GPU stack
could pin it): the last-bit behaviour of ``fp16_tensor / python_int`` on the GPU, which
ATen evaluates as multiply-by-reciprocal.  ``scalar_div='recip'`` restates that rule,
``scalar_div='true'`` is the CPU rule; the GPU test-suite checks the HIP kernels against
torch's own on-device op chain to close the gap.  The accumulation order of ``torch.std_mean`` on the GPU
(last fp16 place of std / mean of the normal-quantile class) is restated in ``std_mean_gpu_tree`` and pinned by
the GPU suite, which compares the HIP quantiser with ``torch.std_mean`` run on the device bit for bit, plus a
known answer recorded from such a run (tests/test_oracle.py).  That pin is to torch on ROCm (MI355X) only: which
order ``torch.std_mean`` takes on the reference's own CUDA platform is covered by no fixture the reference holds, so
the last place of std / mean -- and the sign codes of values next to the mean -- are PARITY UNPINNED against the
reference as its authors ran it.  The CPU order (``NORMAL1_STAT_ORDER = "torch_cpu"``, the default) stays exercised
by the CPU suite.  Also unpinned: the order of equal scores in ``torch.sort`` (block ranking; restated with a stable
sort).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

BITS = (8, 4, 2, 1)   # 1 = the uniform 1-bit class of the 'uniform_group' strategy (qmax 1, 32 codes per word)

# --------------------------------------------------------------------------- pack / unpack


def pack_along_last_dim(data: torch.Tensor, bit: int) -> torch.Tensor:
    """word[..., j] = OR_i (q[..., j*pf+i] << (i*bit)), LSB first, int32.

    Follows quant/pack_unpack.py:40-51 (Triton ``_pack_along_last_dim``) and the
    wrapper at :53-70.
    """
    pf = 32 // bit
    assert data.dtype == torch.int32 and data.shape[-1] % pf == 0
    q = data.reshape(*data.shape[:-1], data.shape[-1] // pf, pf).to(torch.int64)
    word = torch.zeros(q.shape[:-1], dtype=torch.int64)
    for i in range(pf):
        word |= (q[..., i] & ((1 << 32) - 1)) << (i * bit)
    word &= (1 << 32) - 1
    # reinterpret the unsigned 32-bit payload as int32 (the sign bit is just payload)
    word = torch.where(word >= (1 << 31), word - (1 << 32), word)
    return word.to(torch.int32)


def unpack_codes(code: torch.Tensor, bit: int) -> torch.Tensor:
    """Integer codes ``(word >> i*bit) & (0xFF >> (8-bit))`` as int32, last dim * pf.

    quant/pack_unpack.py:272-278.
    """
    pf = 32 // bit
    mask = 0xFF >> (8 - bit)
    w = code.to(torch.int64) & ((1 << 32) - 1)
    shifts = torch.arange(pf, dtype=torch.int64) * bit
    c = (w.unsqueeze(-1) >> shifts) & mask
    return c.reshape(*code.shape[:-1], code.shape[-1] * pf).to(torch.int32)


def unpack_along_last_dim(code: torch.Tensor, bit: int) -> torch.Tensor:
    """Codes stored as fp16 (quant/pack_unpack.py:281-295)."""
    return unpack_codes(code, bit).to(torch.float16)


# --------------------------------------------------------------------------- quantise


def _div_scalar_fp16(x: torch.Tensor, divisor: int, scalar_div: str) -> torch.Tensor:
    """``fp16_tensor / python_int``.

    'recip': what ATen's GPU true-divide does for a CPU scalar divisor -- the fp32
    reciprocal is formed first, then an fp32 multiply, then one rounding to fp16.
    'true' : fp32 divide then one rounding to fp16 (the CPU rule).
    """
    xf = x.to(torch.float32)
    if scalar_div == "recip":
        inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(divisor), dtype=torch.float32)
        return (xf * inv).to(torch.float16)
    if scalar_div == "true":
        return (xf / float(divisor)).to(torch.float16)
    raise ValueError("scalar_div must be 'recip' or 'true'")


def uniform_group_quantize_pack_last_dim(
    data: torch.Tensor, group_size: int, bit: int, scalar_div: str = "recip"
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Asymmetric min/max group quantiser over the last dim; quant/pack_unpack.py:156-193.

    fp16 op chain, each arrow one rounding to fp16:
      mn, mx -> (mx - mn) -> / qmax -> scale ;  x - mn -> / scale -> clamp -> round-half-even
    A group with mx == mn gives 0/0 = NaN, which the GPU's float->int conversion turns
    into code 0; the oracle states that explicitly.  Does not mutate ``data``.
    """
    B, nh, D, T = data.shape
    assert data.dtype == torch.float16 and T % group_size == 0
    qmax = 2 ** bit - 1
    g = data.reshape(B * nh * D, T // group_size, group_size).clone()
    mn = g.min(dim=-1, keepdim=True)[0]
    mx = g.max(dim=-1, keepdim=True)[0]
    scale = _div_scalar_fp16(mx - mn, qmax, scalar_div)
    v = (g - mn) / scale                      # fp16 subtract, fp16 divide (each rounded once)
    v = v.clamp(0, qmax).round()
    v = torch.nan_to_num(v, nan=0.0)
    q = v.to(torch.int32).reshape(B, nh, D, T)
    code = pack_along_last_dim(q, bit)
    shp = (B, nh, D, T // group_size)
    return code, scale.reshape(shp), mn.reshape(shp)


def uniform_group_dequantize_unpack_last_dim(
    code: torch.Tensor, scale: torch.Tensor, mn: torch.Tensor, group_size: int, bit: int
) -> torch.Tensor:
    """x = rnd16(rnd16(fp16(c) * scale) + mn); quant/pack_unpack.py:316-333."""
    B, nh, D, Td = code.shape
    T = Td * (32 // bit)
    x = unpack_along_last_dim(code, bit).reshape(B, nh, D, T // group_size, group_size)
    x = x * scale.unsqueeze(-1)
    x = x + mn.unsqueeze(-1)
    return x.reshape(B, nh, D, T)


# --------------------------------------------------------------------------- 1-bit normal-quantile class
# quant/pack_unpack.py:6-14 for n = 1: upper bounds norm.ppf([0.5, 1.0]) = [0, inf], centres
# norm.ppf([0.25, 0.75]) = -+0.6744897501960817 (fp32), used in the group's dtype: fp16 0.67431640625.
NORMAL1_CENTER = 0.6744897501960817


# How the 1-bit class's statistics are accumulated.  "torch_cpu": ``torch.std_mean`` as this host evaluates it.
# "gpu_tree": the order torch's GPU reduction uses for a 32-element row, which is what the reference runs
# (its quantiser executes on the GPU): the two differ in the last fp16 place of std in rare groups.
NORMAL1_STAT_ORDER = "torch_cpu"


def std_mean_gpu_tree(g: torch.Tensor):
    """std, mean of the last axis (32 fp16 values) in the order of torch's GPU reduction kernel, restated from
    ATen (third party, torch==2.7.1 pinned at requirements.txt:114; native/SharedReduceOps.h ``WelfordOps`` and
    native/cuda/Reduce.cuh): a row of 32 is reduced by 32 threads holding one element each (mean = x, M2 = 0),
    then by shuffles over distances 1, 2, 4, 8, 16, i.e. a balanced tree over ADJACENT halves a (lower indices)
    and b with ``WelfordOps::combine`` in fp32:
        delta = mean_b - mean_a;  mean = mean_a + delta * (n_b / n);  M2 = M2_a + M2_b + delta * delta * n_a * (n_b / n)
    (n_b / n = 1/2 exactly), then ``project``: std = sqrt(M2 / (32 - 1)), both rounded to fp16.
    Pinned by comparing the HIP quantiser, which follows the same order, with ``torch.std_mean`` executed on the
    GPU, bit for bit (tests/test_quant_gpu.py)."""
    mean = g.float()
    m2 = torch.zeros_like(mean)
    n_half = 1.0
    while mean.shape[-1] > 1:
        ma, mb = mean[..., 0::2], mean[..., 1::2]
        delta = mb - ma
        mean = ma + delta * 0.5
        m2 = (m2[..., 0::2] + m2[..., 1::2]) + ((delta * delta) * n_half) * 0.5
        n_half *= 2.0
    # The square root through float64: correctly rounded to fp32 whatever the host (torch.sqrt on fp32 was seen
    # one unit in the last place off on an AVX-512 host, which flips the fp16 rounding of a std that lies next to
    # a rounding boundary; the GPU's sqrt is the correctly rounded one).
    std = torch.sqrt((m2 / 31.0).double()).float()
    return std.to(g.dtype), mean.to(g.dtype)


def normal_group_quantize_pack_last_dim(data: torch.Tensor, group_size: int, bit: int = 1):
    """quant/pack_unpack.py:218-253 for bit == 1: ``std, mean = torch.std_mean(group)`` (unbiased, fp32
    accumulation, rounded to fp16), ``v = rnd16(rnd16(x - mean) / std)``, code = searchsorted([0, inf], v)
    = [v > 0]; packed 32 codes per word.  A NaN (0/0 of a constant group) is stored as code 0 (the reference
    would index past its 2-entry tables)."""
    assert bit == 1, "only the 1-bit table is on the path"
    B, nh, D, T = data.shape
    assert data.dtype == torch.float16 and T % group_size == 0
    g = data.reshape(B * nh * D, T // group_size, group_size)
    if NORMAL1_STAT_ORDER == "gpu_tree" and group_size == 32:
        std, mean = std_mean_gpu_tree(g)
    else:
        std, mean = torch.std_mean(g, dim=-1, keepdim=True)
    v = (g - mean) / std
    q = (v > 0).to(torch.int32).reshape(B, nh, D, T)
    shp = (B, nh, D, T // group_size)
    return pack_along_last_dim(q, 1), std.reshape(shp), mean.reshape(shp)


def normal_group_dequantize_unpack_last_dim(code, std, mean, group_size: int, bit: int = 1):
    """quant/pack_unpack.py:356-376 for bit == 1: x = rnd16(rnd16(centre[c] * std) + mean), the centre in
    the group's dtype."""
    assert bit == 1
    B, nh, D, Td = code.shape
    T = Td * 32
    c = unpack_codes(code, 1).reshape(B, nh, D, T // group_size, group_size).to(torch.int64)
    center = torch.tensor([-NORMAL1_CENTER, NORMAL1_CENTER], dtype=torch.float32)
    x = center[c].to(std.dtype)
    x = x * std.unsqueeze(-1)
    x = x + mean.unsqueeze(-1)
    return x.reshape(B, nh, D, T)


def uniform_group_fake_quant(data: torch.Tensor, group_size: int, bit: int, scalar_div: str = "recip"):
    """quant/pack_unpack.py:134-154 (quantise then dequantise without packing)."""
    if bit == 0:
        return 0
    code, s, z = uniform_group_quantize_pack_last_dim(data, group_size, bit, scalar_div)
    return uniform_group_dequantize_unpack_last_dim(code, s, z, group_size, bit)


# --------------------------------------------------------------------------- GEMV


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(B, Hkv, a, b) -> (B, Hkv*n_rep, a, b), each KV head repeated n_rep times in place.

    transformers' ``repeat_kv`` as used at quant/quant_matmul_hq.py:19,81.
    """
    if n_rep == 1:
        return x
    B, H, a, b = x.shape
    return x[:, :, None].expand(B, H, n_rep, a, b).reshape(B, H * n_rep, a, b)


LOW_NORMAL_STRATEGY = "high_uniform_group_low_normal_group"


def class_quantize(x, bits: int, scalar_div: str = "recip", low_normal: bool = False):
    """The quantiser a class uses: uniform for 8/4/2 bit; for 1 bit uniform under 'uniform_group' and
    normal-quantile under 'high_uniform_group_low_normal_group' (quant/hqe_2.py:482-492)."""
    if bits == 1 and low_normal:
        return normal_group_quantize_pack_last_dim(x, 32, 1)
    return uniform_group_quantize_pack_last_dim(x, 32, bits, scalar_div)


def class_dequantize(code, s, z, bits: int, low_normal: bool = False):
    if bits == 1 and low_normal:
        return normal_group_dequantize_unpack_last_dim(code, s, z, 32, 1)
    return uniform_group_dequantize_unpack_last_dim(code, s, z, 32, bits)


def gemv_uniform_group(group_size, fA, qB, scales, zeros, bits) -> torch.Tensor:
    """C[b,hq,m,n] = sum_k fA[b,hq,m,k] * dq(qB)[b,hq//n_rep,k,n], fp32 accumulate, fp16 out.

    The reference's definition of a correct ``cuda_bmm_fA_qB_uniform_group``
    (quant/matmul.py:263-299): dequantise with the library's own unpack, ``repeat_kv``,
    ``torch.matmul`` (quant/cuda_hq_test.py:82,242; quant/matmul.py:819-832).
    """
    n_rep = fA.shape[1] // qB.shape[1]
    dq = uniform_group_dequantize_unpack_last_dim(qB, scales, zeros, group_size, bits)
    return torch.matmul(fA.float(), repeat_kv(dq, n_rep).float()).to(torch.float16)


# --------------------------------------------------------------------------- hybrid attention

# slot bases of the 42-field cache tuple (quant/quant_matmul_hq.py:34-38)
K16, K16_IDX, V16, V16_IDX = 0, 1, 2, 3
K_BASE = {8: 4, 4: 12, 2: 20, 1: 28}
V_BASE = {8: 8, 4: 16, 2: 24, 1: 32}
V_TOKEN_NORM, NEW_K, NEW_V, KV_SEQ_LEN = 38, 39, 40, 41


def empty_cache(new_K=None, new_V=None, kv_seq_len=0) -> tuple:
    """``(None,)*39 + (K, V, len)`` -- the cache right after prefill (model/llama_hqe.py:186)."""
    return (None,) * 39 + (new_K, new_V, kv_seq_len)


def _scale_clamp_softmax(w: torch.Tensor, head_dim: int, mask, scalar_div: str) -> torch.Tensor:
    """quant/quant_matmul_hq.py:100-103: ``/= sqrt(D)`` (fp16), ``+= mask`` (fp16),
    ``max(., finfo.min)``, fp32 softmax, round to fp16."""
    if scalar_div == "recip":
        inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(head_dim ** 0.5, dtype=torch.float32)
        w = (w.float() * inv).to(torch.float16)
    else:
        w = (w.float() / (head_dim ** 0.5)).to(torch.float16)
    if mask is not None:
        w = w + mask
    w = torch.max(w, torch.tensor(torch.finfo(torch.float16).min, dtype=torch.float16))
    return torch.softmax(w.float(), dim=-1).to(torch.float16)


def qkv_matmul(
    q: torch.Tensor,
    past_key_value: tuple,
    attention_mask,
    head_dim: int,
    quant_strategy: str = "uniform_group",
    block_size: int = 32,
    group_size: int = 32,
    *,
    use_mask: bool = True,
    scalar_div: str = "recip",
    round_per_class: bool = True,
):
    """Hybrid decode attention over the 42-tuple: quant/quant_matmul_hq.py:23-120 and
    quant/hqe_matmul.py:354-451 (``use_mask=False`` restates the latter, which skips the mask).

    ``round_per_class=True`` keeps the reference's ``attn_output +=`` in fp16 after every
    class; ``False`` accumulates every class in fp32 and rounds once (what a fused kernel does).
    Under 'uniform_group' the 1-bit class is a uniform class like the others (quant/hqe_matmul.py:375-377);
    under 'high_uniform_group_low_normal_group' it is the normal-quantile class (:371-374).
    """
    if quant_strategy not in ("uniform_group", "high_uniform_group_low_normal_group"):
        raise ValueError("invalid quant_strategy")
    pkv = past_key_value
    low_normal = quant_strategy == LOW_NORMAL_STRATEGY
    new_K, new_V = pkv[NEW_K], pkv[NEW_V]
    B, Hq, _, D = q.shape
    real_len = 0
    nh_kv = None
    if pkv[V16] is not None:
        nh_kv = pkv[V16].shape[1]
        real_len += pkv[V16].shape[2]
    for b in BITS:
        v = pkv[V_BASE[b]]
        if v is not None:
            nh_kv = v.shape[1]
            real_len += v.shape[2]
    new_len = 0
    if new_V is not None:
        nh_kv = new_V.shape[1]
        new_len = new_V.shape[2]
        real_len += new_len
    if real_len == 0:
        raise ValueError("invalid past_key_value")
    n_rep = Hq // nh_kv
    w = torch.zeros(B, Hq, 1, real_len, dtype=torch.float16)
    if pkv[K16] is not None:
        w[..., pkv[K16_IDX]] = torch.matmul(q.float(), repeat_kv(pkv[K16], n_rep).float()).half()
    for b in BITS:
        base = K_BASE[b]
        if pkv[base] is not None:
            dqk = class_dequantize(pkv[base], pkv[base + 2], pkv[base + 3], b, low_normal)
            w[..., pkv[base + 1]] = torch.matmul(q.float(), repeat_kv(dqk, n_rep).float()).to(torch.float16)
    if new_K is not None:
        w[..., real_len - new_len:] = torch.matmul(
            q.float(), repeat_kv(new_K, n_rep).transpose(2, 3).float()).half()
    w = _scale_clamp_softmax(w, head_dim, attention_mask if use_mask else None, scalar_div)

    acc32 = torch.zeros(B, Hq, 1, D, dtype=torch.float32)
    acc16 = torch.zeros(B, Hq, 1, D, dtype=torch.float16)

    def _add(part32):
        nonlocal acc32, acc16
        acc32 = acc32 + part32
        acc16 = acc16 + part32.half()

    if pkv[V16] is not None:
        _add(torch.matmul(w[..., pkv[V16_IDX]].float(), repeat_kv(pkv[V16], n_rep).float()))
    for b in BITS:
        base = V_BASE[b]
        if pkv[base] is not None:
            dq = class_dequantize(pkv[base], pkv[base + 2], pkv[base + 3], b, low_normal)
            _add(torch.matmul(w[..., pkv[base + 1]].float(), repeat_kv(dq, n_rep).float()))
    if new_V is not None:
        _add(torch.matmul(w[..., real_len - new_len:].float(), repeat_kv(new_V, n_rep).float()))
    out = acc16 if round_per_class else acc32.half()
    return w, out


# --------------------------------------------------------------------------- policy helpers


def calculate_token_range(new_cache: Optional[torch.Tensor], token_range: Optional[torch.Tensor]):
    """Per-token sum over (batch, head) of max_d - min_d, appended to the running vector.
    model/public_func.py:58-73."""
    if new_cache is None:
        return None
    r = (new_cache.max(dim=-1)[0] - new_cache.min(dim=-1)[0]).sum(0).sum(0)
    return r if token_range is None else torch.cat((token_range, r), dim=-1)


def get_block_token_idx(block_size: int, block_num: int, importance: torch.Tensor) -> torch.Tensor:
    """Token indices of 32-token blocks ordered by descending mean importance.
    model/public_func.py:92-106 (the in-place divide of the caller's tensor is not reproduced)."""
    bi = importance.reshape(block_num, -1)
    bi = (bi / bi.shape[1]).sum(dim=-1)
    _, order = torch.sort(bi, descending=True, stable=True)
    return (order.reshape(-1, 1) * block_size + torch.arange(block_size, dtype=order.dtype)).flatten()


def make_sum_equal(array: torch.Tensor, array_sum: int, start_idx: int = 4) -> torch.Tensor:
    """Repair rounded block counts so they sum to ``array_sum`` (model/public_func.py:259-268): a surplus is
    taken from index ``start_idx`` and then from the indices below it, none below zero; a deficit is added to
    index ``start_idx``.  Returns a repaired copy."""
    a = [int(x) for x in array.tolist()]
    surplus = sum(a) - int(array_sum)
    if surplus < 0:
        a[start_idx] -= surplus
    for i in range(start_idx, -1, -1):
        if surplus <= 0:
            break
        cut = min(a[i], surplus)
        a[i] -= cut
        surplus -= cut
    return torch.tensor(a, dtype=array.dtype)


def rerank_after_eviction(idx_per_class: Sequence[Optional[torch.Tensor]]) -> List[Optional[torch.Tensor]]:
    """Replace every surviving position by its rank among all survivors (quant/hqe_2.py:661-670).
    Written with a Python dict instead of the reference's all-pairs compare."""
    alive = sorted(int(v) for t in idx_per_class if t is not None for v in t.tolist())
    rank = {v: r for r, v in enumerate(alive)}
    out = []
    for t in idx_per_class:
        out.append(None if t is None else torch.tensor([rank[int(v)] for v in t.tolist()], dtype=torch.int64))
    return out


# --------------------------------------------------------------------------- cache policy (unit lists)
#
# Restatement of KV_cache_hqe_2 (quant/hqe_2.py:456-843) and KV_cache_compress
# (quant/hybrid_quant.py:318-612) on explicit lists of units instead of concatenated tensors:
# a K unit is one 32-token group of one class (the granularity at which the reference moves K,
# quant/hqe_2.py:102-117), a V unit is one token.  The quantiser is local to a group, so quantising
# unit by unit equals the reference's batched calls; class tensors are the units concatenated in
# list order, which is the reference's torch.cat order.  Slow by design (Python loops).

_CLASS_BITS = (16, 8, 4, 2, 1)


def _units_from_class(data, idx, scale, zero, bits, is_k):
    units = []
    if data is None:
        return units
    if is_k:
        n = idx.numel()
        assert n % 32 == 0
        pf = 32 // bits if bits < 16 else 1
        for g in range(n // 32):
            u = dict(idx=idx[32 * g:32 * g + 32].clone(), bits=bits)
            if bits == 16:
                u["x"] = data[..., 32 * g:32 * g + 32].clone()
            else:
                w = 32 // pf
                u["x"] = (data[..., w * g:w * g + w].clone(), scale[..., g:g + 1].clone(), zero[..., g:g + 1].clone())
            units.append(u)
    else:
        for t in range(idx.numel()):
            u = dict(idx=idx[t:t + 1].clone(), bits=bits)
            if bits == 16:
                u["x"] = data[:, :, t:t + 1, :].clone()
            else:
                u["x"] = (data[:, :, t:t + 1, :].clone(), scale[:, :, t:t + 1, :].clone(), zero[:, :, t:t + 1, :].clone())
            units.append(u)
    return units


def _unit_fp16(u, low_normal=False):
    if u["bits"] == 16:
        return u["x"]
    c, s, z = u["x"]
    return class_dequantize(c, s, z, u["bits"], low_normal)


def _unit_requant(u, bits, scalar_div, low_normal=False):
    x = _unit_fp16(u, low_normal)
    if bits == 16:
        return dict(idx=u["idx"], bits=16, x=x)
    return dict(idx=u["idx"], bits=bits, x=class_quantize(x, bits, scalar_div, low_normal))


def _class_from_units(units, bits, is_k):
    if not units:
        return (None, None) if bits == 16 else (None, None, None, None)
    idx = torch.cat([u["idx"] for u in units])
    dim = 3 if is_k else 2
    if bits == 16:
        return torch.cat([u["x"] for u in units], dim=dim), idx
    return (torch.cat([u["x"][0] for u in units], dim=dim), idx,
            torch.cat([u["x"][1] for u in units], dim=dim), torch.cat([u["x"][2] for u in units], dim=dim))


def _policy_side(pkv, new, history, sorted_idx, bit_num, is_k, scalar_div, low_normal=False):
    """-> ({bits: units}, surviving positions before re-ranking or None if nothing was to be evicted)."""
    slots = K_BASE if is_k else V_BASE
    cls = {}
    for b in _CLASS_BITS:
        if b == 16:
            cls[b] = _units_from_class(pkv[K16 if is_k else V16], pkv[K16_IDX if is_k else V16_IDX], None, None, 16, is_k)
        else:
            s = slots[b]
            cls[b] = _units_from_class(pkv[s], pkv[s + 1], pkv[s + 2], pkv[s + 3], b, is_k)
    # new tokens as units (K: in 32-token groups that are formed at the moment they move)
    n_new = new.shape[2]
    new_tokens = [dict(idx=torch.tensor([history + t]), x=new[:, :, t:t + 1, :]) for t in range(n_new)]
    cum = [0] + torch.cumsum(bit_num.to(torch.int64), 0).tolist()
    target = [set(sorted_idx[cum[i]:cum[i + 1]].tolist()) for i in range(len(cum) - 1)]
    has_evict = len(target) > 5 and len(target[5]) > 0
    if has_evict:
        new_tokens = [u for u in new_tokens if int(u["idx"][0]) not in target[5]]
        for b in _CLASS_BITS:
            kept = []
            for u in cls[b]:
                hit = [int(v) in target[5] for v in u["idx"].tolist()]
                assert all(hit) or not any(hit), "a unit is evicted as a whole"
                if not hit[0]:
                    kept.append(u)
            cls[b] = kept
    survivors = None
    if has_evict:
        survivors = sorted([int(v) for b in _CLASS_BITS for u in cls[b] for v in u["idx"].tolist()]
                           + [int(u["idx"][0]) for u in new_tokens])
    for ti in (4, 3, 2, 1, 0):
        tb, tset = _CLASS_BITS[ti], target[ti]
        if not tset:
            continue
        moved = [u for u in new_tokens if int(u["idx"][0]) in tset]
        if moved:
            new_tokens = [u for u in new_tokens if int(u["idx"][0]) not in tset]
            if is_k:
                assert len(moved) % 32 == 0
                for g in range(len(moved) // 32):
                    grp = moved[32 * g:32 * g + 32]
                    x = torch.cat([u["x"] for u in grp], dim=2).transpose(2, 3).contiguous()   # (B,H,D,32)
                    cls[tb].append(_unit_requant(dict(idx=torch.cat([u["idx"] for u in grp]), bits=16, x=x), tb, scalar_div, low_normal))
            else:
                for u in moved:
                    cls[tb].append(_unit_requant(dict(idx=u["idx"], bits=16, x=u["x"]), tb, scalar_div, low_normal))
        for sb in _CLASS_BITS:
            if sb <= tb:
                break
            stay = []
            for u in cls[sb]:
                hit = [int(v) in tset for v in u["idx"].tolist()]
                assert all(hit) or not any(hit)
                if hit[0]:
                    cls[tb].append(_unit_requant(u, tb, scalar_div, low_normal))
                else:
                    stay.append(u)
            cls[sb] = stay
    assert not new_tokens, "every new token is assigned to a class or evicted"
    if len(target) > 5 and (cum[6] > cum[5]):
        rank = {v: r for r, v in enumerate(sorted(int(v) for b in _CLASS_BITS for u in cls[b] for v in u["idx"].tolist()))}
        for b in _CLASS_BITS:
            for u in cls[b]:
                u["idx"] = torch.tensor([rank[int(v)] for v in u["idx"].tolist()], dtype=torch.int64)
    return cls, survivors


def compress_cache(past_key_value: tuple, compress_length: int, history_length: int, K_sorted_idx, K_bit_num,
                   V_bit_num, token_importance, *, times_range: bool = True, scalar_div: str = "recip",
                   weights_ring: Optional[torch.Tensor] = None, quant_strategy: str = "uniform_group"):
    """One compression step; 6-entry bit_num = KV_cache_hqe_2, 5-entry = KV_cache_compress.
    Returns (new 42-tuple, ring of recent attention rows after eviction or None).  The 1-bit class is the
    uniform one under 'uniform_group' and the normal-quantile one under
    'high_uniform_group_low_normal_group' (quant/hqe_2.py:482-492)."""
    pkv = past_key_value
    low_normal = quant_strategy == LOW_NORMAL_STRATEGY
    new_K, new_V = pkv[NEW_K], pkv[NEW_V]
    res_K = new_K[:, :, compress_length:, :].clone()
    res_V = new_V[:, :, compress_length:, :].clone()
    new_K, new_V = new_K[:, :, :compress_length, :], new_V[:, :, :compress_length, :]
    total = history_length + compress_length
    V_norm = calculate_token_range(new_V, pkv[V_TOKEN_NORM])
    V_score = token_importance * V_norm if times_range else token_importance.clone()
    V_sorted_idx = get_block_token_idx(32, total // 32, V_score)
    k_cls, _ = _policy_side(pkv, new_K, history_length, K_sorted_idx, K_bit_num, True, scalar_div, low_normal)
    v_cls, v_alive = _policy_side(pkv, new_V, history_length, V_sorted_idx, V_bit_num, False, scalar_div, low_normal)
    if v_alive is not None:
        keep = torch.tensor(v_alive, dtype=torch.int64)
        V_norm = V_norm[keep]
        if weights_ring is not None:
            weights_ring = weights_ring.clone()
            kept = weights_ring[:, keep]
            weights_ring[:, :kept.shape[1]] = kept
    t = [None] * 42
    t[K16], t[K16_IDX] = _class_from_units(k_cls[16], 16, True)
    t[V16], t[V16_IDX] = _class_from_units(v_cls[16], 16, False)
    for b in BITS:
        s = K_BASE[b]
        t[s], t[s + 1], t[s + 2], t[s + 3] = _class_from_units(k_cls[b], b, True)
        s = V_BASE[b]
        t[s], t[s + 1], t[s + 2], t[s + 3] = _class_from_units(v_cls[b], b, False)
    t[V_TOKEN_NORM] = V_norm
    t[NEW_K] = res_K if res_K.numel() else None
    t[NEW_V] = res_V if res_V.numel() else None
    t[KV_SEQ_LEN] = pkv[KV_SEQ_LEN]
    return tuple(t), weights_ring


def reconstruct_cache(past_key_value: tuple, quant_strategy: str = "uniform_group"):
    """Dense fp16 (K, V) (B,H,kv_seq_len,D) from the tuple (quant/hybrid_quant.py:732-846, with the 4-bit V
    class restored unconditionally)."""
    pkv = past_key_value
    low_normal = quant_strategy == LOW_NORMAL_STRATEGY
    T = int(pkv[KV_SEQ_LEN])
    ref = next(x for x in (pkv[NEW_V], pkv[V16]) if x is not None) if (pkv[NEW_V] is not None or pkv[V16] is not None) else None
    if ref is not None:
        B, H, D = ref.shape[0], ref.shape[1], ref.shape[3]
    else:
        b = next(b for b in BITS if pkv[V_BASE[b]] is not None)
        B, H, D = pkv[V_BASE[b]].shape[0], pkv[V_BASE[b]].shape[1], pkv[V_BASE[b]].shape[3] * (32 // b)
    K = torch.zeros(B, H, T, D, dtype=torch.float16)
    V = torch.zeros(B, H, T, D, dtype=torch.float16)
    if pkv[K16] is not None:
        K[:, :, pkv[K16_IDX]] = pkv[K16].transpose(2, 3)
    if pkv[V16] is not None:
        V[:, :, pkv[V16_IDX]] = pkv[V16]
    for b in BITS:
        s = K_BASE[b]
        if pkv[s] is not None:
            K[:, :, pkv[s + 1]] = class_dequantize(pkv[s], pkv[s + 2], pkv[s + 3], b, low_normal).transpose(2, 3)
        s = V_BASE[b]
        if pkv[s] is not None:
            V[:, :, pkv[s + 1]] = class_dequantize(pkv[s], pkv[s + 2], pkv[s + 3], b, low_normal)
    if pkv[NEW_K] is not None:
        K[:, :, T - pkv[NEW_K].shape[2]:] = pkv[NEW_K]
        V[:, :, T - pkv[NEW_V].shape[2]:] = pkv[NEW_V]
    return K, V


# --------------------------------------------------------------------------- the layer that calls the path
class ImportanceRing:
    """model/public_func.py:208-257: the last ``last_length`` attention rows, each summed over the batch and
    then over the heads in the rows' own dtype; a prompt fills the store from the top with its last rows, a
    decode step writes the row at ``next_line`` and moves on, modulo ``last_length``.
    importance[j] = column sum / number of stored rows that have seen token j."""

    def __init__(self, last_length: int = 20, max_length: int = 0):
        self.last_length, self.max_length = last_length, max_length
        self.kv_seq_len = 0
        self.next_line = 0
        self.weights = None

    def update(self, attn_weights: torch.Tensor) -> None:
        if self.weights is None:
            self.weights = torch.zeros(self.last_length, self.max_length, dtype=attn_weights.dtype)
        L, T = attn_weights.shape[2], attn_weights.shape[3]
        rows = min(L, self.last_length) if L > 1 else 1
        summed = attn_weights[:, :, L - rows:, :].sum(0).sum(0)            # (rows, T)
        first = 0 if L > 1 else self.next_line
        self.weights[first:first + rows, :T] = summed
        self.kv_seq_len = T
        self.next_line = (self.next_line + rows) % self.last_length

    def importance(self) -> torch.Tensor:
        n = self.kv_seq_len
        seen = torch.tensor([min(self.last_length, n - j) for j in range(n)], dtype=self.weights.dtype)
        return self.weights[:, :n].sum(0) / seen


class DecodeLayerOracle:
    """The cache-side state machine of ``LlamaAttention_hqe.forward`` (model/llama_hqe.py:55-251) without
    the projections, the rotary embedding and ``o_proj``: prefill builds ``(None,)*39 + (K, V, len)``
    (:186), a decode step appends to ``new_K/new_V`` (:131-133) and attends over the tuple (:136), every
    call feeds the ring (:199) and, once 32 un-quantised tokens exist, derives the class sizes (:216-224),
    ranks blocks (:228), compresses (:230-231) and rescales the ratios for the next increment (:233-239).
    ``observed`` lets a test feed the ring with another implementation's probabilities so that both walk
    through identical policy decisions."""

    def __init__(self, head_dim: int, bit_0: float, bit_4: float, bit_2: float, bit_1: float = 0.0,
                 times_range: bool = True, last_length: int = 20, max_length: int = 0, scalar_div: str = "recip",
                 quant_strategy: str = "uniform_group"):
        self.head_dim = head_dim
        self.quant_strategy = quant_strategy
        self.times_range = times_range
        self.scalar_div = scalar_div
        self.ratio_e_0 = torch.tensor([bit_0], dtype=torch.float32)
        self.ratio_e = self.ratio_e_0.clone()
        self.ratio_q = torch.tensor([bit_4, bit_2, bit_1], dtype=torch.float32)
        self.current_length = 0
        self.history_reserve_length = 0
        self.ring = ImportanceRing(last_length, max_length)

    def step(self, q, k, v, attention_mask=None, past_key_value=None, auxiliary_parameters=None, observed=None):
        """q (B,Hq,L,D), k/v (B,Hkv,L,D) after rotary.  Returns (attn_output (B,Hq,L,D) fp16,
        attn_weights, new tuple, auxiliary_parameters)."""
        L = k.shape[-2]
        self.current_length += L
        kv_seq_len = L + (past_key_value[-1] if past_key_value is not None else 0)
        if past_key_value is not None:
            new_K = torch.cat((past_key_value[-3], k), dim=2) if past_key_value[-3] is not None else k
            new_V = torch.cat((past_key_value[-2], v), dim=2) if past_key_value[-2] is not None else v
            past_key_value = past_key_value[:-3] + (new_K, new_V, kv_seq_len)
            attn_weights, attn_output = qkv_matmul(q, past_key_value, attention_mask, self.head_dim,
                                                   self.quant_strategy, use_mask=False, scalar_div=self.scalar_div)
        else:
            n_rep = q.shape[1] // k.shape[1]
            w = torch.matmul(q.float(), repeat_kv(k, n_rep).transpose(2, 3).float()).half()
            w = (w.float() * (self.head_dim ** -0.5)).half()
            if attention_mask is not None:
                w = w + attention_mask
                w = torch.max(w, torch.tensor(torch.finfo(torch.float16).min, dtype=torch.float16))
            attn_weights = torch.softmax(w.float(), dim=-1).half()
            attn_output = torch.matmul(attn_weights.float(), repeat_kv(v, n_rep).float()).half()
            past_key_value = (None,) * 39 + (k, v, kv_seq_len)

        self.ring.update(attn_weights if observed is None else observed)
        if self.current_length < 32:
            return attn_output, attn_weights, past_key_value, None
        compress_length = self.current_length - self.current_length % 32
        total = self.history_reserve_length + compress_length
        if auxiliary_parameters is not None:      # sized by layer 0 of the same step (:211-214)
            compress_ratio, K_bit_num, V_bit_num = auxiliary_parameters
        else:
            compress_ratio, K_bit_num = split_history(total, self.ratio_q, self.ratio_e)
            V_bit_num = K_bit_num.clone()
        importance = self.ring.importance()[:total]
        K_token_idx = get_block_token_idx(32, total // 32, importance)
        # the reference's ranking helper divides its argument by the block length in place
        # (model/public_func.py:94-96), so its policy receives importance / 32 (model/llama_hqe.py:226-231)
        past_key_value, ring = compress_cache(past_key_value, compress_length, self.history_reserve_length,
                                              K_token_idx, K_bit_num, V_bit_num, importance / 32,
                                              times_range=self.times_range, scalar_div=self.scalar_div,
                                              weights_ring=self.ring.weights,
                                              quant_strategy=self.quant_strategy)
        if ring is not None:
            self.ring.weights = ring
        self.history_reserve_length += compress_length - int(K_bit_num[-1])
        self.current_length -= compress_length
        if auxiliary_parameters is None:
            # (:235-239) the eviction share is meant for the tokens the next compression adds
            add = (self.history_reserve_length + 32) // 32 * 32 - self.history_reserve_length
            self.ratio_e = (add * self.ratio_e_0) / (self.history_reserve_length + add)
            self.ratio_q = (1 - self.ratio_e) * self.ratio_q / self.ratio_q.sum()
        return attn_output, attn_weights, past_key_value, (compress_ratio, K_bit_num, V_bit_num)


def split_history(total: int, ratio_q: torch.Tensor, ratio_e: torch.Tensor):
    """model/llama_hqe.py:216-224: float32 shares of (fp16, 8, 4, 2, 1 bit, evicted) -- 64 tokens fp16, no
    8-bit class, the remainder by ``ratio_q`` and ``ratio_e`` -- turned into whole 32-token blocks by rounding
    and ``make_sum_equal``.  -> (shares, tokens per target as int32)."""
    fp16_share = torch.tensor([64 / total, 0], dtype=torch.float32)
    shares = torch.cat((fp16_share, ratio_q, ratio_e))
    shares[2:] = (1 - shares[0]) * shares[2:]
    blocks = total // 32
    return shares, make_sum_equal(torch.round(blocks * shares).to(torch.int), blocks) * 32


class KiviLayerOracle:
    """The cache-side logic of the reference's KIVI-style attention (model/llama_kivi.py:96-266) without the
    projections, the rotary embedding and ``o_proj``: every token is kept, K is quantised per channel in
    blocks of ``residual_length`` tokens once that many fp16 tokens have gathered (:155-167,236-252), V per
    token, one token at a time, as soon as more than ``residual_length`` fp16 tokens exist (:190-203,254-264).
    Cache tuple (:266): (K codes (B,H,D,Tq/pf), K fp16 tail (B,H,r,D), K scale, K zero, V codes (B,H,Tv,D/pf),
    V fp16 tail, V scale, V zero, kv_seq_len).  A decode step attends over the quantised part with the
    per-class GEMV and over the fp16 tails with plain matmuls (:130-188); here both run as dequantise-then-
    matmul, the reference's own definition of the GEMV's result (quant/cuda_hq_test.py:82,242)."""

    def __init__(self, head_dim: int, k_bits: int = 2, v_bits: int = 2, group_size: int = 32,
                 residual_length: int = 128, scalar_div: str = "recip"):
        assert residual_length % group_size == 0
        self.head_dim, self.k_bits, self.v_bits = head_dim, k_bits, v_bits
        self.group_size, self.residual_length, self.scalar_div = group_size, residual_length, scalar_div

    def _q(self, x, bits):
        return uniform_group_quantize_pack_last_dim(x, self.group_size, bits, self.scalar_div)

    def step(self, q, k, v, attention_mask=None, past_key_value=None, observed=None):
        """-> (attn_output (B,Hq,L,D) fp16, attn_weights fp16, new 9-tuple).  ``observed``: probabilities of
        another implementation for the same decode step; the output is then computed from THEM, which checks
        that implementation's p.V stage on its own (a raw score that lands on the other side of an fp16
        rounding boundary moves a peaked row's probabilities by up to half a percent, and the output with them)."""
        n_rep = q.shape[1] // k.shape[1]
        R, D = self.residual_length, self.head_dim
        kv_seq_len = k.shape[-2] + (past_key_value[-1] if past_key_value is not None else 0)
        if past_key_value is not None:
            kq, k_full, ks, kz, vq, v_full, vs, vz, _ = past_key_value
            att_q = gemv_uniform_group(self.group_size, q, kq, ks, kz, self.k_bits) if kq is not None else None
            k_full = torch.cat([k_full, k], dim=2) if k_full is not None else k
            att_f = torch.matmul(q.float(), repeat_kv(k_full, n_rep).transpose(2, 3).float()).half()
            w = torch.cat([att_q, att_f], dim=-1) if att_q is not None else att_f
            # ``/ sqrt(D)`` in fp16, the mask if any, fp32 softmax (:145-173); the clamp is the identity without a mask
            w = _scale_clamp_softmax(w, D, attention_mask, self.scalar_div)
            w_own = w
            if observed is not None:
                w = observed
            if k_full.shape[-2] == R:
                c, s, z = self._q(k_full.transpose(2, 3).contiguous(), self.k_bits)
                k_full = None
                kq = c if kq is None else torch.cat([kq, c], dim=3)
                ks = s if ks is None else torch.cat([ks, s], dim=3)
                kz = z if kz is None else torch.cat([kz, z], dim=3)
            v_full = torch.cat([v_full, v], dim=2)
            nf = v_full.shape[-2]
            if vq is None:
                out = torch.matmul(w.float(), repeat_kv(v_full, n_rep).float()).half()
            else:
                out = gemv_uniform_group(self.group_size, w[..., :-nf], vq, vs, vz, self.v_bits)
                out = out + torch.matmul(w[..., -nf:].float(), repeat_kv(v_full, n_rep).float()).half()
            if nf > R:
                c, s, z = self._q(v_full[:, :, :1, :].contiguous(), self.v_bits)
                v_full = v_full[:, :, 1:, :].contiguous()
                vq = c if vq is None else torch.cat([vq, c], dim=2)
                vs = s if vs is None else torch.cat([vs, s], dim=2)
                vz = z if vz is None else torch.cat([vz, z], dim=2)
        else:
            T = k.shape[-2]
            w = torch.matmul(q.float(), repeat_kv(k, n_rep).transpose(2, 3).float()).half()
            w = (w.float() * (D ** -0.5)).half()
            if attention_mask is not None:
                w = w + attention_mask
                w = torch.max(w, torch.tensor(torch.finfo(torch.float16).min, dtype=torch.float16))
            w = torch.softmax(w.float(), dim=-1).half()
            out = torch.matmul(w.float(), repeat_kv(v, n_rep).float()).half()
            if T % R != 0:
                if T < R:
                    k_quant, k_full = None, k
                else:
                    k_quant, k_full = k[:, :, :-(T % R), :].contiguous(), k[:, :, -(T % R):, :].contiguous()
            else:
                k_quant, k_full = k, None
            kq = ks = kz = None
            if k_quant is not None:
                kq, ks, kz = self._q(k_quant.transpose(2, 3).contiguous(), self.k_bits)
            if T <= R:
                vq, v_full, vs, vz = None, v, None, None
            else:
                v_full = v[:, :, -R:, :].contiguous()
                vq, vs, vz = self._q(v[:, :, :-R, :].contiguous(), self.v_bits)
        return out, (w_own if past_key_value is not None else w), (kq, k_full, ks, kz, vq, v_full, vs, vz, kv_seq_len)
