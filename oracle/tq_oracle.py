"""CPU oracle for the TurboQuant KV-cache path.  TEST INFRASTRUCTURE ONLY.

This module restates, op for op, what the reference's pure-PyTorch CPU path
computes for the TQ4 compress / decompress / fused attention / paged decode
operators and for the host-side set-up they consume (codebook, rotation,
packing, TurboQuantMSE / TurboQuantProd).  It is the checker for the HIP
kernels: only tests, the smoke check and the benchmark's CPU-baseline leg may
import it.  Nothing in the shipped package may call it.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  The arithmetic lives in PyTorch CPU ops exactly as in
the reference (``torch.norm``, ``@``, ``torch.bucketize``, ``torch.softmax``,
``torch.linalg.qr``, ``torch.randn``); the reference's own tests pin those
only through tolerances and properties, so at the last-bit level the floating
point results are "parity unpinned" and are pinned at the stated tolerances
(index mismatch <= 1e-4, relative MSE <= 1e-3, attention max-abs <= 2e-2).

Pinned by (see tests/test_oracle_*.py):
  nibble_pack / nibble_unpack / pack_2bit / unpack_2bit
      known answers of tests/test_packing.py:46-64 and
      csrc/tests/test_packing.cpp:22-28, all 256 byte values by brute force.
  lloyd_max_gaussian
      fixed point of the Lloyd map in float64, antisymmetry, midpoints,
      distortion of the textbook 16-level Gaussian quantizer.
  haar_orthogonal
      orthogonality, determinism, sign rule; committed fixture for drift.
  compress / decompress
      scalar pure-Python brute force on tiny inputs, range/finite invariants.
  attention / fused_tq_attention
      torch.nn.functional.scaled_dot_product_attention, rotated-space identity.
  paged_decode_loop / paged_decode_gather
      each other, block-table permutation invariance, SDPA over gathered rows.
  paged_prefill
      fused_tq_attention on the same tokens (one page run per sequence, full
      queries), paged_decode_gather for one query per sequence, SDPA with an
      explicit bottom-right mask for a chunked prefill.
  prod_quantize / prod_inner_product
      sign/zero rule; with the identity as sketch the correction term equals
      gamma * sqrt(pi/2)/d * <q, sign(residual)> exactly; its mean over 400
      sketches is <q, residual> / sqrt(d) (the reference's normalisation,
      core/quantizer.py:264-268, 355-370, reproduced as is); the gain over
      many keys; explicit sums.  A dropped, halved or doubled term fails these.
  prod_paged_decode
      against explicit prod_inner_product scores + softmax + mse_dequantize
      values through the packed page; the page layout itself is parity
      unpinned (the reference has no paged TurboQuantProd path).
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

TQ4_LEVELS = 16
NORM_BYTES = 4  # src/flashquant/vllm/spec.py:30


# ---------------------------------------------------------------------------
# Set-up: codebook and rotation
# ---------------------------------------------------------------------------


def lloyd_max_gaussian(dim: int, bits: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Lloyd-Max levels for N(0, 1/dim) truncated to +-3.5 sigma.

    Follows src/flashquant/core/codebook.py:58-140: uniform start on the
    support, at most 200 sweeps of (midpoint boundaries, conditional means) in
    float64 with the outer edges fixed at +-3.5 sigma, stop when the largest
    centroid move is below 1e-10, return float32 (centroids, boundaries).
    """
    levels = 1 << bits
    sigma = 1.0 / math.sqrt(dim)
    lo, hi = -3.5 * sigma, 3.5 * sigma
    cent = torch.tensor(
        [lo + (hi - lo) * (i + 0.5) / levels for i in range(levels)],
        dtype=torch.float64,
    )
    inv_sigma = 1.0 / sigma
    erf_scale = inv_sigma / math.sqrt(2.0)
    pdf_scale = 1.0 / (sigma * math.sqrt(2.0 * math.pi))

    def pdf(t: torch.Tensor) -> torch.Tensor:
        return pdf_scale * torch.exp(-0.5 * (t * inv_sigma) ** 2)

    def cdf(t: torch.Tensor) -> torch.Tensor:
        return 0.5 * (1.0 + torch.erf(t * erf_scale))

    lo_t = torch.tensor([lo], dtype=torch.float64)
    hi_t = torch.tensor([hi], dtype=torch.float64)
    for _ in range(200):
        mid = (cent[:-1] + cent[1:]) / 2.0
        edges = torch.cat([lo_t, mid, hi_t])
        a, b = edges[:-1], edges[1:]
        mass = cdf(b) - cdf(a)
        ok = mass > 1e-15
        mean = (sigma ** 2) * (pdf(a) - pdf(b)) / torch.where(ok, mass, torch.ones_like(mass))
        new = torch.where(ok, mean, (a + b) / 2.0)
        shift = (new - cent).abs().max().item()
        cent = new
        if shift < 1e-10:
            break
    bnd = (cent[:-1] + cent[1:]) / 2.0
    return cent.float(), bnd.float()


def haar_orthogonal(dim: int, seed: int = 42) -> torch.Tensor:
    """Seeded Haar rotation (src/flashquant/core/quantizer.py:60-85).

    CPU generator, float32 Gaussian matrix, QR, columns of Q multiplied by the
    sign of diag(R) with zero mapped to +1.
    """
    gen = torch.Generator(device="cpu").manual_seed(seed)
    g = torch.randn(dim, dim, generator=gen, device="cpu", dtype=torch.float32)
    q, r = torch.linalg.qr(g)
    s = torch.sign(torch.diag(r))
    s[s == 0] = 1.0
    return q * s.unsqueeze(0)


def qjl_matrix(dim: int, seed: int = 42, qjl_dim: Optional[int] = None) -> torch.Tensor:
    """Gaussian sketch S / sqrt(m), generator seeded with seed + 1
    (src/flashquant/core/quantizer.py:264-268)."""
    m = qjl_dim or dim
    gen = torch.Generator(device="cpu").manual_seed(seed + 1)
    s = torch.randn(m, dim, generator=gen, device="cpu", dtype=torch.float32)
    return s / math.sqrt(m)


def split_rotation(rotation: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Even / odd columns of rotation.T, contiguous
    (src/flashquant/kernels/compress.py:86-89, csrc/core/rotation.cpp:41-61)."""
    rt = rotation.T.contiguous()
    return rt[:, 0::2].contiguous(), rt[:, 1::2].contiguous()


# ---------------------------------------------------------------------------
# Packing (integer, bit-exact)
# ---------------------------------------------------------------------------


def nibble_pack(indices: torch.Tensor) -> torch.Tensor:
    """byte j = idx[2j] << 4 | idx[2j+1] (src/flashquant/core/packing.py:54-79;
    the range / parity errors are those of tests/conftest.py:224-234)."""
    if indices.shape[-1] % 2 != 0:
        raise ValueError(
            f"Last dimension must be even for nibble packing, got {indices.shape[-1]}"
        )
    if indices.numel() and (int(indices.max()) > 15 or int(indices.min()) < 0):
        raise ValueError("Values > 15 cannot be packed into 4-bit nibbles")
    hi = indices[..., 0::2].to(torch.uint8)
    lo = indices[..., 1::2].to(torch.uint8)
    return (hi << 4) | lo


def nibble_unpack(packed: torch.Tensor) -> torch.Tensor:
    """Inverse of nibble_pack, int64, high nibble first
    (src/flashquant/core/packing.py:82-98)."""
    hi = (packed >> 4).long()
    lo = (packed & 0x0F).long()
    return torch.stack([hi, lo], dim=-1).flatten(-2)


def pack_2bit(indices: torch.Tensor) -> torch.Tensor:
    """Four 2-bit values per byte, first value in the top bits
    (csrc/core/packing.cpp:48-64, tests/conftest.py:244-256)."""
    d = indices.shape[-1]
    if d % 4 != 0:
        raise ValueError(f"Last dim must be divisible by 4, got {d}")
    if indices.numel() and (int(indices.max()) > 3 or int(indices.min()) < 0):
        raise ValueError("Values > 3 cannot be packed into 2 bits")
    v = indices.to(torch.uint8)
    return (v[..., 0::4] << 6) | (v[..., 1::4] << 4) | (v[..., 2::4] << 2) | v[..., 3::4]


def unpack_2bit(packed: torch.Tensor) -> torch.Tensor:
    """Inverse of pack_2bit, int64 (csrc/core/packing.cpp:66-79)."""
    parts = [((packed >> s) & 0x03).long() for s in (6, 4, 2, 0)]
    return torch.stack(parts, dim=-1).flatten(-2)


# ---------------------------------------------------------------------------
# TQ4 compress / decompress
# ---------------------------------------------------------------------------


def compress(
    x: torch.Tensor, rotation: torch.Tensor, boundaries: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """TQ4 compress (src/flashquant/kernels/cpu_reference.py:22-61).

    x (N, H, D) any float dtype -> packed (N, H, D/2) uint8, norms (N, H, 1)
    float32.  Steps: float32 rows; L2 norm; divide by (norm + 1e-10);
    multiply by rotation.T; bucketize (count of boundaries strictly below the
    value); clamp to [0, 15]; nibble pack with the even coordinate on top.
    """
    n, h, d = x.shape
    rows = x.reshape(n * h, d).float()
    norms = torch.norm(rows, dim=-1, keepdim=True)
    unit = rows / (norms + 1e-10)
    y = unit @ rotation.T
    idx = torch.bucketize(y, boundaries).clamp(0, TQ4_LEVELS - 1).to(torch.uint8)
    packed = (idx[:, 0::2] << 4) | idx[:, 1::2]
    return packed.reshape(n, h, d // 2), norms.reshape(n, h, 1)


def compress_indices(
    x: torch.Tensor, rotation: torch.Tensor, boundaries: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Same computation as compress() but also returns the rotated unit
    vectors, for tests that need the distance of a coordinate to its nearest
    boundary when judging index mismatches."""
    n, h, d = x.shape
    rows = x.reshape(n * h, d).float()
    norms = torch.norm(rows, dim=-1, keepdim=True)
    y = (rows / (norms + 1e-10)) @ rotation.T
    idx = torch.bucketize(y, boundaries).clamp(0, TQ4_LEVELS - 1)
    return idx.reshape(n, h, d), norms.reshape(n, h, 1), y.reshape(n, h, d)


def decompress(
    packed: torch.Tensor, norms: torch.Tensor, centroids: torch.Tensor
) -> torch.Tensor:
    """TQ4 decompress (src/flashquant/kernels/cpu_reference.py:64-94).

    packed (N, H, D/2) uint8, norms (N, H, 1) float32 -> (N, H, D) float32 in
    rotated space: coordinate 2j comes from the high nibble of byte j and
    2j+1 from the low nibble; value = centroid * norm in float32.  The
    dispatcher casts to the requested dtype afterwards
    (src/flashquant/kernels/decompress.py:80-86).
    """
    n, h, half = packed.shape
    idx = torch.stack([(packed >> 4).long(), (packed & 0x0F).long()], dim=-1)
    idx = idx.reshape(n * h, 2 * half)
    vals = centroids[idx] * norms.reshape(n * h, 1)
    return vals.reshape(n, h, 2 * half)


# ---------------------------------------------------------------------------
# Attention
# ---------------------------------------------------------------------------


def attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    sm_scale: Optional[float] = None,
    is_causal: bool = False,
) -> torch.Tensor:
    """Dense attention (src/flashquant/kernels/cpu_reference.py:97-151).

    q (B, HQ, NQ, D), k/v (B, HKV, NKV, D).  KV heads are repeated to the
    query head count, scores are float32, the causal mask hides k > q counted
    from the top-left corner, and the mask is dropped when NQ == 1.  Result is
    cast to q.dtype.
    """
    b, hq, nq, d = q.shape
    hkv, nkv = k.shape[1], k.shape[2]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    if nq == 1:
        is_causal = False
    if hq != hkv:
        rep = hq // hkv
        k = k.repeat_interleave(rep, dim=1)
        v = v.repeat_interleave(rep, dim=1)
    s = torch.matmul(q.float(), k.float().transpose(-2, -1)) * sm_scale
    if is_causal:
        hide = torch.triu(torch.ones(nq, nkv, dtype=torch.bool), diagonal=1)
        s = s.masked_fill(hide[None, None], float("-inf"))
    w = torch.softmax(s, dim=-1)
    return torch.matmul(w, v.float()).to(q.dtype)


def fused_tq_attention(
    q: torch.Tensor,
    k_packed: torch.Tensor,
    k_norms: torch.Tensor,
    v_packed: torch.Tensor,
    v_norms: torch.Tensor,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    rotation: torch.Tensor,
    sm_scale: Optional[float] = None,
    is_causal: bool = False,
) -> torch.Tensor:
    """Fused TQ4 attention as the dispatcher computes it on CPU, from the
    un-rotated query to the output in the original space
    (src/flashquant/kernels/attention.py:85-107 and
    src/flashquant/kernels/cpu_reference.py:154-227).

    q_rot = (q.float() @ R.T).to(q.dtype); K and V are decompressed in rotated
    space; attention() runs on them (its result is cast to q.dtype); the
    result is multiplied by R in float32 and cast to q.dtype again.
    """
    b, hq, nq, d = q.shape
    hkv, nkv, half = k_packed.shape[1], k_packed.shape[2], k_packed.shape[3]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    q_rot = torch.matmul(q.float(), rotation.T).to(q.dtype)
    k = decompress(k_packed.reshape(b * hkv, nkv, half), k_norms.reshape(b * hkv, nkv, 1), centroids_k)
    v = decompress(v_packed.reshape(b * hkv, nkv, half), v_norms.reshape(b * hkv, nkv, 1), centroids_v)
    k = k.reshape(b, hkv, nkv, d)
    v = v.reshape(b, hkv, nkv, d)
    # cpu_reference.py:194 hands attention() the float32 view of q_rot, so the
    # rotated-space result is float32 there and is only cast once, after the
    # multiplication by R (cpu_reference.py:226).
    out_rot = attention(q_rot.float(), k, v, sm_scale=sm_scale, is_causal=is_causal)
    return torch.matmul(out_rot.float(), rotation).to(q.dtype)


# ---------------------------------------------------------------------------
# Packed paged cache: layout, store, decode
# ---------------------------------------------------------------------------


def page_layout(num_kv_heads: int, head_dim: int) -> Tuple[int, int, int, int]:
    """Byte offsets inside one token row of the packed cache
    (src/flashquant/vllm/impl.py:132-138):
    [K indices H*D/2 | K norms H*4 | V indices H*D/2 | V norms H*4].
    Returns (k_norm_off, v_idx_off, v_norm_off, row_bytes)."""
    half = head_dim // 2
    k_norm_off = num_kv_heads * half
    v_idx_off = k_norm_off + num_kv_heads * NORM_BYTES
    v_norm_off = v_idx_off + num_kv_heads * half
    return k_norm_off, v_idx_off, v_norm_off, v_norm_off + num_kv_heads * NORM_BYTES


def store_rows(
    kv_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    k_packed: torch.Tensor,
    k_norms: torch.Tensor,
    v_packed: torch.Tensor,
    v_norms: torch.Tensor,
) -> None:
    """Row assembly and scatter into the paged cache
    (src/flashquant/vllm/impl.py:243-263): the float32 norms are stored as
    their four little-endian bytes; slot = block * block_size + row."""
    n, h, half = k_packed.shape
    k_norm_off, v_idx_off, v_norm_off, row_bytes = page_layout(h, 2 * half)
    row = torch.empty(n, row_bytes, dtype=torch.uint8)
    row[:, :k_norm_off] = k_packed.reshape(n, -1)
    row[:, k_norm_off:v_idx_off] = k_norms.reshape(n, h).contiguous().view(torch.uint8)
    row[:, v_idx_off:v_norm_off] = v_packed.reshape(n, -1)
    row[:, v_norm_off:] = v_norms.reshape(n, h).contiguous().view(torch.uint8)
    flat = kv_cache.view(-1, row_bytes)
    flat[slot_mapping.long()] = row


def paged_decode_loop(
    q_rot: torch.Tensor,
    kv_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
    sm_scale: Optional[float] = None,
) -> torch.Tensor:
    """Token-by-token paged decode in rotated space
    (src/flashquant/kernels/cpu_reference.py:230-368).  For small cases only.

    q_rot (S, HQ, D) already rotated; returns (S, HQ, D) in q_rot.dtype,
    rotated space; a sequence of length 0 yields zeros.
    """
    s_count, hq, d = q_rot.shape
    half = head_dim // 2
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    k_norm_off, v_idx_off, v_norm_off, _ = page_layout(num_kv_heads, head_dim)
    out = torch.zeros_like(q_rot)
    rep = hq // num_kv_heads
    for s in range(s_count):
        length = int(seq_lens[s])
        if length == 0:
            continue
        k_rows = torch.empty(num_kv_heads, length, head_dim)
        v_rows = torch.empty(num_kv_heads, length, head_dim)
        for t in range(length):
            page = int(block_table[s, t // block_size])
            row = kv_cache[page, t % block_size]
            for h in range(num_kv_heads):
                kb = row[h * half:(h + 1) * half]
                kn = row[k_norm_off + 4 * h:k_norm_off + 4 * h + 4].clone().view(torch.float32)
                vb = row[v_idx_off + h * half:v_idx_off + (h + 1) * half]
                vn = row[v_norm_off + 4 * h:v_norm_off + 4 * h + 4].clone().view(torch.float32)
                k_rows[h, t] = centroids_k[nibble_unpack(kb)] * kn
                v_rows[h, t] = centroids_v[nibble_unpack(vb)] * vn
        if rep > 1:
            k_rows = k_rows.repeat_interleave(rep, dim=0)
            v_rows = v_rows.repeat_interleave(rep, dim=0)
        qs = q_rot[s].float()
        sc = torch.bmm(qs.unsqueeze(1), k_rows.transpose(-2, -1)) * sm_scale
        w = torch.softmax(sc, dim=-1)
        out[s] = torch.bmm(w, v_rows).squeeze(1).to(q_rot.dtype)
    return out


def gather_sequence(
    kv_cache: torch.Tensor,
    block_table_row: torch.Tensor,
    length: int,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dequantised K, V (H, length, D) float32 of one sequence, gathered
    through its block-table row with vectorised indexing.  Same values as the
    inner loops of paged_decode_loop."""
    half = head_dim // 2
    k_norm_off, v_idx_off, v_norm_off, row_bytes = page_layout(num_kv_heads, head_dim)
    t = torch.arange(length)
    pages = block_table_row.long()[t // block_size]
    rows = kv_cache.view(-1, row_bytes)[pages * block_size + (t % block_size)]
    kb = rows[:, :k_norm_off].reshape(length, num_kv_heads, half)
    kn = rows[:, k_norm_off:v_idx_off].contiguous().view(torch.float32).reshape(length, num_kv_heads, 1)
    vb = rows[:, v_idx_off:v_norm_off].reshape(length, num_kv_heads, half)
    vn = rows[:, v_norm_off:].contiguous().view(torch.float32).reshape(length, num_kv_heads, 1)
    k = decompress(kb, kn, centroids_k).permute(1, 0, 2).contiguous()
    v = decompress(vb, vn, centroids_v).permute(1, 0, 2).contiguous()
    return k, v


def paged_decode_gather(
    q_rot: torch.Tensor,
    kv_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
    sm_scale: Optional[float] = None,
) -> torch.Tensor:
    """paged_decode_loop with the per-token Python loops replaced by one
    gather per sequence; the softmax / matmul sequence is unchanged."""
    s_count, hq, d = q_rot.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    out = torch.zeros_like(q_rot)
    rep = hq // num_kv_heads
    for s in range(s_count):
        length = int(seq_lens[s])
        if length == 0:
            continue
        k, v = gather_sequence(kv_cache, block_table[s], length, centroids_k, centroids_v,
                               num_kv_heads, head_dim, block_size)
        if rep > 1:
            k = k.repeat_interleave(rep, dim=0)
            v = v.repeat_interleave(rep, dim=0)
        sc = torch.bmm(q_rot[s].float().unsqueeze(1), k.transpose(-2, -1)) * sm_scale
        w = torch.softmax(sc, dim=-1)
        out[s] = torch.bmm(w, v).squeeze(1).to(q_rot.dtype)
    return out


def split_k_paged_decode(
    q: torch.Tensor,
    kv_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    rotation: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
    sm_scale: Optional[float] = None,
    faithful_loop: bool = False,
) -> torch.Tensor:
    """The dispatcher's CPU path from un-rotated q to original-space output
    (src/flashquant/kernels/paged_decode.py:112-128): rotate q and cast to
    q.dtype, decode in rotated space (cast to q.dtype), multiply by R in
    float32, cast to q.dtype."""
    q_rot = torch.matmul(q.float(), rotation.T).to(q.dtype)
    fn = paged_decode_loop if faithful_loop else paged_decode_gather
    out_rot = fn(q_rot, kv_cache, block_table, seq_lens, centroids_k, centroids_v,
                 num_kv_heads, head_dim, block_size, sm_scale=sm_scale)
    return torch.matmul(out_rot.float(), rotation).to(q.dtype)


def paged_prefill(
    q: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    kv_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    rotation: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
    sm_scale: Optional[float] = None,
    causal: bool = True,
) -> torch.Tensor:
    """Prefill over the packed paged cache as the serving backend computes it
    (src/flashquant/vllm/impl.py:317-336 and 470-512): the queries of all
    sequences are packed along the token axis, q (T, HQ, D); q_rot =
    (q.float() @ R.T).to(q.dtype); the cache is decompressed in rotated space
    to q.dtype (impl.py:298-305); a variable-length attention over
    (cu_seqlens_q, seq_lens, block_table) gives a q.dtype result, which is
    multiplied by R in float32 and cast to q.dtype (impl.py:506-510).

    The attention call itself belongs to vllm's flash-attention library, which
    is not in the reference checkout; its published semantics are restated:
    float32 scores and softmax, a causal mask aligned to the bottom-right
    corner (query j of n sees keys 0 .. L - n + j), result cast to q.dtype.
    """
    total, hq, d = q.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    rep = hq // num_kv_heads
    q_rot = torch.matmul(q.float(), rotation.T).to(q.dtype)
    out_rot = torch.zeros_like(q_rot)
    for s in range(seq_lens.shape[0]):
        first, end = int(cu_seqlens_q[s]), int(cu_seqlens_q[s + 1])
        n, length = end - first, int(seq_lens[s])
        if n == 0 or length == 0:
            continue
        k, v = gather_sequence(kv_cache, block_table[s], length, centroids_k, centroids_v,
                               num_kv_heads, head_dim, block_size)
        k = k.to(q.dtype).float()
        v = v.to(q.dtype).float()
        if rep > 1:
            k = k.repeat_interleave(rep, dim=0)
            v = v.repeat_interleave(rep, dim=0)
        qs = q_rot[first:end].float().permute(1, 0, 2)                 # (HQ, n, D)
        sc = torch.bmm(qs, k.transpose(-2, -1)) * sm_scale             # (HQ, n, L)
        if causal:
            key_pos = torch.arange(length)[None, :]
            q_pos = (length - n + torch.arange(n))[:, None]
            sc = sc.masked_fill((key_pos > q_pos)[None], float("-inf"))
        w = torch.softmax(sc, dim=-1)
        out_rot[first:end] = torch.bmm(w, v).permute(1, 0, 2).to(q.dtype)
    return torch.matmul(out_rot.float(), rotation).to(q.dtype)


# ---------------------------------------------------------------------------
# TurboQuantMSE / TurboQuantProd (arbitrary bit width)
# ---------------------------------------------------------------------------


def mse_quantize(
    x: torch.Tensor, rotation: torch.Tensor, boundaries: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """TurboQuantMSE.quantize (src/flashquant/core/quantizer.py:145-159):
    indices (..., D) int64 (not clamped), norms (..., 1) float32."""
    d = x.shape[-1]
    rows = x.reshape(-1, d).float()
    norms = torch.norm(rows, dim=-1, keepdim=True)
    y = (rows / (norms + 1e-10)) @ rotation.T
    idx = torch.bucketize(y, boundaries)
    return idx.reshape(x.shape), norms.reshape(*x.shape[:-1], 1)


def mse_dequantize(
    indices: torch.Tensor, norms: torch.Tensor, rotation: torch.Tensor, centroids: torch.Tensor
) -> torch.Tensor:
    """TurboQuantMSE.dequantize (src/flashquant/core/quantizer.py:181-195):
    (centroids[idx] @ R) * norm, float32, original space."""
    d = indices.shape[-1]
    rec = centroids[indices.reshape(-1, d)] @ rotation
    return (rec * norms.reshape(-1, 1)).reshape(indices.shape)


def prod_quantize(
    x: torch.Tensor,
    rotation: torch.Tensor,
    boundaries: torch.Tensor,
    centroids: torch.Tensor,
    sketch: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """TurboQuantProd.quantize (src/flashquant/core/quantizer.py:285-304).

    boundaries / centroids are those of the (bits - 1) codebook.  Returns
    (indices, norms, signs, residual_norms); signs are +-1 float32 with a zero
    projection mapped to +1.
    """
    d = x.shape[-1]
    idx, norms = mse_quantize(x, rotation, boundaries)
    resid = x.float() - mse_dequantize(idx, norms, rotation, centroids)
    gamma = torch.norm(resid, dim=-1, keepdim=True)
    proj = resid.reshape(-1, d) @ sketch.T
    signs = torch.sign(proj).reshape(*x.shape[:-1], sketch.shape[0])
    signs[signs == 0] = 1.0
    return idx, norms, signs, gamma


def prod_inner_product(
    query: torch.Tensor,
    indices: torch.Tensor,
    norms: torch.Tensor,
    signs: torch.Tensor,
    residual_norms: torch.Tensor,
    rotation: torch.Tensor,
    centroids: torch.Tensor,
    sketch: torch.Tensor,
) -> torch.Tensor:
    """TurboQuantProd.estimate_inner_product
    (src/flashquant/core/quantizer.py:355-370):
    <q, k_mse> + gamma * sqrt(pi/2) / m * <S q, signs>, shape (..., 1)."""
    d = query.shape[-1]
    m = sketch.shape[0]
    k_mse = mse_dequantize(indices, norms, rotation, centroids)
    first = (query.float() * k_mse).sum(dim=-1, keepdim=True)
    q_proj = (query.float().reshape(-1, d) @ sketch.T).reshape(*query.shape[:-1], m)
    corr = (q_proj * signs).sum(dim=-1, keepdim=True)
    return first + residual_norms * math.sqrt(math.pi / 2.0) / m * corr


# ---------------------------------------------------------------------------
# TurboQuantProd keys + TQ4 values as pages (a composition: the reference has
# the quantizer, src/flashquant/core/quantizer.py:270-370, but no paged path)
# ---------------------------------------------------------------------------


def prod_pack_keys(indices: torch.Tensor, signs: torch.Tensor) -> torch.Tensor:
    """Key nibble = sign_bit << 3 | 3-bit index (sign_bit 1 for a -1 sign),
    packed two per byte like nibble_pack (even coordinate in the high nibble)."""
    nib = indices.long() | ((signs < 0).long() << 3)
    return nibble_pack(nib)


def prod_page_layout(num_kv_heads: int, head_dim: int) -> Tuple[int, int, int, int, int]:
    """Offsets (k_norm, k_gamma, v_idx, v_norm, row_bytes) of the token row
    [K nibbles | K norms | K residual norms | V idx | V norms]."""
    k_norm = num_kv_heads * (head_dim // 2)
    k_gamma = k_norm + NORM_BYTES * num_kv_heads
    v_idx = k_gamma + NORM_BYTES * num_kv_heads
    v_norm = v_idx + num_kv_heads * (head_dim // 2)
    return k_norm, k_gamma, v_idx, v_norm, v_norm + NORM_BYTES * num_kv_heads


def prod_store_rows(kv_cache, slot_mapping, k_packed, k_norms, k_gamma, v_packed, v_norms) -> None:
    n, h, half = k_packed.shape
    k_norm, k_gam, v_idx, v_norm, row_bytes = prod_page_layout(h, 2 * half)
    row = torch.empty(n, row_bytes, dtype=torch.uint8)
    row[:, :k_norm] = k_packed.reshape(n, -1)
    row[:, k_norm:k_gam] = k_norms.reshape(n, h).contiguous().view(torch.uint8)
    row[:, k_gam:v_idx] = k_gamma.reshape(n, h).contiguous().view(torch.uint8)
    row[:, v_idx:v_norm] = v_packed.reshape(n, -1)
    row[:, v_norm:] = v_norms.reshape(n, h).contiguous().view(torch.uint8)
    kv_cache.view(-1, row_bytes)[slot_mapping.long()] = row


def prod_paged_decode(
    q: torch.Tensor,
    kv_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    centroids_k3: torch.Tensor,
    centroids_v: torch.Tensor,
    rotation: torch.Tensor,
    sketch: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
    sm_scale: Optional[float] = None,
) -> torch.Tensor:
    """Decode over TurboQuantProd key / TQ4 value pages.

    Score of a key = TurboQuantProd.estimate_inner_product
    (src/flashquant/core/quantizer.py:355-370): <q, k_mse> + gamma sqrt(pi/2)/m
    <S q, signs>, with <q, k_mse> evaluated in rotated space as norm * <q_rot,
    centroids[idx]> and q_rot = (q @ R.T) rounded to q.dtype as the TQ4 decode
    dispatcher rounds it (src/flashquant/kernels/paged_decode.py:113).  Values are
    TQ4 in rotated space; the result is rounded to q.dtype, multiplied by R and
    rounded again (paged_decode.py:123).  A sequence of length 0 gives zeros.
    """
    s_count, hq, d = q.shape
    m = sketch.shape[0]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    half = head_dim // 2
    k_norm, k_gam, v_idx, v_norm, row_bytes = prod_page_layout(num_kv_heads, head_dim)
    rep = hq // num_kv_heads
    q_rot = torch.matmul(q.float(), rotation.T).to(q.dtype).float()
    q_s = torch.matmul(q.float(), sketch.T)
    out_rot = torch.zeros(s_count, hq, d, dtype=q.dtype)
    for s in range(s_count):
        length = int(seq_lens[s])
        if length == 0:
            continue
        t = torch.arange(length)
        pages = block_table[s].long()[t // block_size]
        rows = kv_cache.view(-1, row_bytes)[pages * block_size + (t % block_size)]
        nib = nibble_unpack(rows[:, :k_norm].reshape(length, num_kv_heads, half))
        idx, sign = nib & 7, 1.0 - 2.0 * (nib >> 3).float()
        kn = rows[:, k_norm:k_gam].contiguous().view(torch.float32).reshape(length, num_kv_heads, 1)
        kg = rows[:, k_gam:v_idx].contiguous().view(torch.float32).reshape(length, num_kv_heads, 1)
        vb = rows[:, v_idx:v_norm].reshape(length, num_kv_heads, half)
        vn = rows[:, v_norm:].contiguous().view(torch.float32).reshape(length, num_kv_heads, 1)
        k_mse = (centroids_k3[idx] * kn).permute(1, 0, 2)                 # (H, L, D), rotated space
        sg = (sign * kg * (math.sqrt(math.pi / 2.0) / m)).permute(1, 0, 2)   # (H, L, m)
        v = decompress(vb, vn, centroids_v).permute(1, 0, 2)
        if rep > 1:
            k_mse = k_mse.repeat_interleave(rep, dim=0)
            sg = sg.repeat_interleave(rep, dim=0)
            v = v.repeat_interleave(rep, dim=0)
        sc = torch.bmm(q_rot[s].unsqueeze(1), k_mse.transpose(-2, -1)) + torch.bmm(q_s[s].unsqueeze(1), sg.transpose(-2, -1))
        w = torch.softmax(sc * sm_scale, dim=-1)
        out_rot[s] = torch.bmm(w, v).squeeze(1).to(q.dtype)
    return torch.matmul(out_rot.float(), rotation).to(q.dtype)
