"""CPU restatement of kernl's three fused operators — TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Two kinds of function live here, each citing the reference file:line it follows (paths relative to the
reference checkout, `src/kernl/...`):

* closed forms in fp32 torch (`attention_oracle`, `linear_oracle`, `layer_norm_oracle`, `rms_norm_oracle`):
  what the reference's own tests compare its Triton kernels against;
* step-by-step restatements of the reference KERNELS in numpy float64/float32 (`attention_tiled_oracle`,
  `layer_norm_welford_oracle`): the tile loop, -inf clamp, online-softmax update and chunked Welford merge exactly
  as the Triton code performs them.  They pin behaviour the closed forms leave open (what a fully masked row
  returns, that the chunked variance equals the two-pass one).

How each function is pinned (tests/test_oracle.py):
  attention_oracle        torch.softmax/matmul closed form; V=1 => O=1; truncating -inf padded keys; causal row 0 = v[0];
                          key-permutation invariance; brute-force scalar loops on tiny inputs
  attention_tiled_oracle  equals attention_oracle on tile-edge sizes (8, 16, 33, 128, 257); fully masked row = mean(V)
  linear_oracle           F.linear closed form; gelu(0)=0, relu(-1)=0, erf/tanh table values; x.mT strided input
  layer_norm_oracle       F.layer_norm; large-mean input (-20 + 0.5 randn); unit-variance closed form
  layer_norm_welford_oracle equals layer_norm_oracle to fp32 rounding for N in {128 .. 4096 .. 5000}
  rms_norm_oracle         x * rsqrt(mean(x^2)+eps) * w closed form; constant-row known answer
  effective_eps           code reading only (layer_norm.py:295-296)
  glu_oracle              (a*sigmoid(a))*b written out as in the reference kernel vs F.silu(F.linear)*F.linear; gate = 0
                          gives 0, value weights = 0 with unit bias gives act(gate)
  rotary_oracle           equals rotary_complex_oracle (the reference's complex product) under the even/odd <-> half
                          permutation; zero angle = identity; angles add; quarter turn of a unit vector; norms kept
  rotary_complex_oracle   torch.view_as_complex product as in the reference; pinned by the same known answers
  embedding_layer_norm_oracle  F.embedding + F.layer_norm with fp32 tables (nothing rounds between the additions); with
                          fp16 tables, F.layer_norm of the sum formed by fp16 tensor additions; one table = plain lookup
                          (tests/test_host_logic.py::test_embedding_oracle_against_the_library_routines)
Nothing here is "parity unpinned".
"""
import math
from typing import Optional

import numpy as np
import torch

ACTIVATION_NAMES = ("", "tanh", "relu", "gelu", "fast_gelu", "silu")


# ------------------------------------------------------------------------------------------------------------------
# attention
# ------------------------------------------------------------------------------------------------------------------
def attention_oracle(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    sm_scale: float,
    is_causal: bool = False,
    attention_mask: Optional[torch.Tensor] = None,
    start_position: int = 0,
) -> torch.Tensor:
    """softmax(q·kᵀ·sm_scale + mask, causal)·v in fp32 on the CPU.

    Follows `attention_reference`, implementations/attention.py:29-61: scale, ADD the mask, set keys n > m to -inf
    when causal (`tril` of an [m, n] matrix, i.e. top-left aligned), softmax over keys, times v.  Inputs of any
    float dtype are upcast to fp32 first; the result is fp32.  `start_position` shifts the causal diagonal: keys
    n > m + start_position are masked, the `triu(..., diagonal=start_pos + 1)` mask of
    experimental/llama-v2/llama/model.py:338-343 (pinned in tests/test_oracle.py by the rows start_position.. of a
    top-left aligned causal attention over the whole sequence).
    """
    q32, k32, v32 = q.detach().float().cpu(), k.detach().float().cpu(), v.detach().float().cpu()
    p = torch.matmul(q32, k32.transpose(-1, -2)) * sm_scale
    if attention_mask is not None:
        p = p + attention_mask.detach().float().cpu()
    if is_causal:
        m_size, n_size = q32.size(-2), k32.size(-2)
        keep = torch.tril(torch.ones((m_size, n_size), dtype=torch.bool), diagonal=start_position)
        p = torch.where(keep, p, torch.tensor(float("-inf")))
    p = torch.softmax(p, dim=-1)
    return torch.matmul(p, v32)


def attention_tiled_oracle(
    q: np.ndarray,
    k: np.ndarray,
    v: np.ndarray,
    sm_scale: float,
    is_causal: bool = False,
    attention_mask: Optional[np.ndarray] = None,
    min_clamp_value: Optional[float] = None,
    block_m: int = 128,
    block_n: int = 128,
) -> np.ndarray:
    """The reference KERNEL's algorithm, tile by tile, in float64 numpy (implementations/attention.py:238-435).

    q [B,H,M,D], k/v [B,H,N,D]; mask [B|1,H|1,M|1,N] additive.  Per (128-row query block, batch·head):
      * loop over 128-key blocks up to n (or up to (block_m_idx+1)·128 when causal, :304-309);
      * qk = q·kᵀ·sm_scale (:344-345); causal adds -inf where m < n (:346-347); keys beyond n are -inf (:342-343);
      * mask entries equal to -inf are replaced by `min_clamp_value` = finfo(mask dtype).min before the add
        (:380, host side :516), so a fully masked row stays finite;
      * online softmax with a NORMALISED accumulator (:390-429): l_new = max(l_i, l_j), alpha = exp(l_i - l_new),
        beta = exp(l_j - l_new), d_new = alpha d_i + beta d_j, P = numerators·beta/d_new,
        acc = acc·(d_i/d_new·alpha) + P·v.
    """
    B, H, M, D = q.shape
    N = k.shape[2]
    out = np.zeros((B, H, M, D), dtype=np.float64)
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    if attention_mask is not None:
        if min_clamp_value is None:
            min_clamp_value = float(np.finfo(attention_mask.dtype).min)
        mask64 = attention_mask.astype(np.float64)
        mask64 = np.where(np.isneginf(mask64), min_clamp_value, mask64)
    for b in range(B):
        for h in range(H):
            for m0 in range(0, M, block_m):
                m1 = min(m0 + block_m, M)
                rows = np.arange(m0, m1)
                l_i = np.full((m1 - m0,), -np.inf)
                d_i = np.zeros((m1 - m0,))
                acc = np.zeros((m1 - m0, D))
                n_end = N
                if is_causal:
                    n_end = (m0 // block_m + 1) * block_n
                for n0 in range(0, n_end, block_n):
                    cols = np.arange(n0, n0 + block_n)
                    valid = cols < N
                    kk = np.zeros((block_n, D))
                    vv = np.zeros((block_n, D))
                    kk[valid] = k64[b, h, cols[valid]]
                    vv[valid] = v64[b, h, cols[valid]]
                    qk = q64[b, h, m0:m1] @ kk.T * sm_scale
                    qk[:, ~valid] = -np.inf
                    if is_causal:
                        qk = qk + np.where(rows[:, None] >= cols[None, :], 0.0, -np.inf)
                    if attention_mask is not None:
                        mb = b if attention_mask.shape[0] != 1 else 0
                        mh = h if attention_mask.shape[1] != 1 else 0
                        mm = np.full((m1 - m0, block_n), -np.inf)  # out-of-range loads return -inf (:372-377) ...
                        if attention_mask.shape[2] == 1:
                            mm[:, valid] = mask64[mb, mh, 0, cols[valid]][None, :]
                        else:
                            mm[:, valid] = mask64[mb, mh, m0:m1][:, cols[valid]]
                        mm = np.where(np.isneginf(mm), min_clamp_value, mm)  # ... and are clamped like the rest
                        with np.errstate(invalid="ignore"):
                            qk = qk + mm
                    l_j = qk.max(axis=1)
                    with np.errstate(invalid="ignore"):
                        numerators = np.exp(qk - l_j[:, None])
                        d_j = numerators.sum(axis=1)
                        l_new = np.maximum(l_i, l_j)
                        alpha = np.exp(l_i - l_new)
                        beta = np.exp(l_j - l_new)
                        d_new = alpha * d_i + beta * d_j
                        p_scale = beta / d_new
                        acc = acc * (d_i / d_new * alpha)[:, None] + (numerators * p_scale[:, None]) @ vv
                    d_i, l_i = d_new, l_new
                out[b, h, m0:m1] = acc
    return out


# ------------------------------------------------------------------------------------------------------------------
# linear + activations
# ------------------------------------------------------------------------------------------------------------------
def activation_oracle(x: torch.Tensor, activation: str) -> torch.Tensor:
    """Activations of implementations/activation_func.py:28-49 on an fp32 tensor: "tanh", "relu",
    "fast_gelu" = 0.5x(1+tanh(sqrt(2/pi)(x+0.044715x^3))), "gelu" = 0.5x(1+erf(x/sqrt 2)).  "silu" (x·sigmoid x) is
    this build's addition.  Any other name is the identity, as in linear_layer.py:198-205."""
    if activation == "tanh":
        return torch.tanh(x)
    if activation == "relu":
        return torch.clamp_min(x, 0.0)
    if activation == "fast_gelu":
        return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x * x * x)))
    if activation == "gelu":
        return x * 0.5 * (1.0 + torch.erf(x / math.sqrt(2.0)))
    if activation == "silu":
        return x * torch.sigmoid(x)
    return x


def linear_oracle(
    x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], activation: str = "", return_act_inputs: bool = False
):
    """activation(x @ weightᵀ + bias) in fp32 (implementations/linear_layer.py:92-210: fp32 accumulator initialised
    with the bias :174-178, activation on the accumulator :198-205; weight is [N, K])."""
    x32, w32 = x.detach().float().cpu(), weight.detach().float().cpu()
    pre = x32 @ w32.transpose(-1, -2)
    if bias is not None:
        pre = pre + bias.detach().float().cpu()
    out = activation_oracle(pre, activation)
    return (out, pre) if return_act_inputs else out


# ------------------------------------------------------------------------------------------------------------------
# layer norm
# ------------------------------------------------------------------------------------------------------------------
def glu_oracle(
    x: torch.Tensor,
    w_gate: torch.Tensor,
    b_gate: Optional[torch.Tensor],
    w_value: torch.Tensor,
    b_value: Optional[torch.Tensor],
    activation: str = "silu",
) -> torch.Tensor:
    """act(x·w_gateᵀ + b_gate) * (x·w_valueᵀ + b_value) in fp32: the product the reference's fused feed-forward
    forms from its two accumulators, `(acc1 * sigmoid(acc1)) * acc2`
    (experimental/llama-v2/kernel/fused_kernel_ff.py:36-75, eager form llama/model.py `FeedForward.forward`)."""
    gate = linear_oracle(x, w_gate, b_gate, activation)
    return gate * linear_oracle(x, w_value, b_value, "")


def effective_eps(eps: float, dtype: torch.dtype) -> float:
    """eps the reference actually uses: clamped to >= 1.6e-5 for fp16 inputs (implementations/layer_norm.py:295-296)."""
    return max(eps, 1.6e-5) if dtype == torch.float16 else eps


def layer_norm_oracle(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """(x - mean)/sqrt(biased var + eps)·w + b over the last dim, fp32 (implementations/layer_norm.py:182-205)."""
    x32 = x.detach().float().cpu()
    mean = x32.mean(dim=-1, keepdim=True)
    var = ((x32 - mean) ** 2).mean(dim=-1, keepdim=True)
    out = (x32 - mean) / torch.sqrt(var + eps) * weight.detach().float().cpu()
    if bias is not None:
        out = out + bias.detach().float().cpu()
    return out


def embedding_layer_norm_oracle(tables, ids, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """LayerNorm of the sum of embedding lookups, the rows added in the tables' dtype one after the other as an eager
    model adds them (`word + token_type`, then `+ position`: transformers' BertEmbeddings.forward; the reference runs
    these as PyTorch ops in front of its LayerNorm kernel, implementations/layer_norm.py:115-205).  ids broadcast
    against each other; the result is fp32."""
    dtype = tables[0].dtype
    shape = torch.broadcast_shapes(*[tuple(i.shape) for i in ids])
    total = None
    for table, index in zip(tables, ids):
        rows = table.detach().cpu()[index.detach().cpu().expand(shape)]
        total = rows if total is None else (total.float() + rows.float()).to(dtype)
    return layer_norm_oracle(total, weight, bias, eps)


def rms_norm_oracle(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x·rsqrt(mean(x²)+eps)·w, fp32 (implementations/layer_norm.py:41-57 and the IS_RMSNORM branch :169-170,:182-183)."""
    x32 = x.detach().float().cpu()
    variance = x32.pow(2).mean(-1, keepdim=True)
    return x32 * torch.rsqrt(variance + eps) * weight.detach().float().cpu()


def layer_norm_welford_oracle(
    x: np.ndarray, weight: np.ndarray, bias: Optional[np.ndarray], eps: float, use_rms_norm: bool = False,
    block_n_size: Optional[int] = None,
):
    """The reference KERNEL, chunk by chunk, in fp32 numpy (implementations/layer_norm.py:152-205).

    Row-wise: for each chunk of BLOCK_N_SIZE columns compute block_mean, block_delta = Σ(a - block_mean)·a, then
    merge with the running (mean, var) by Chan's rule with the term delta²·(n_prev·n_blk)/n_tot (:159-180);
    `var /= N`, `rstd = 1/sqrt(var + eps)`; RMS keeps mean = 0 and accumulates Σa² (:169-170).
    BLOCK_N_SIZE defaults to the host heuristic clamp(next_pow2(N), 128, 4096) (:306-311).
    Returns (out, mean, rstd).
    """
    x = x.astype(np.float32)
    M, N = x.shape
    if block_n_size is None:
        block_n_size = min(max(1 << max(N - 1, 0).bit_length(), 128), 4096)
    out = np.empty_like(x)
    means = np.zeros((M,), dtype=np.float32)
    rstds = np.zeros((M,), dtype=np.float32)
    for row in range(M):
        mean = np.float32(0.0)
        var = np.float32(0.0)
        for start in range(0, N, block_n_size):
            end = min(start + block_n_size, N)
            a = x[row, start:end]
            cnt = np.float32(end - start)
            if use_rms_norm:
                var += np.sum(a * a, dtype=np.float32)
            else:
                block_mean = np.sum(a, dtype=np.float32) / cnt
                delta_mean = block_mean - mean
                block_delta = np.sum((a - block_mean) * a, dtype=np.float32)
                mean = mean + np.sum(a - mean, dtype=np.float32) / np.float32(end)
                var = var + block_delta + delta_mean * delta_mean * np.float32(start) * cnt / np.float32(end)
        var = var / np.float32(N)
        rstd = np.float32(1.0) / np.sqrt(var + np.float32(eps))
        means[row], rstds[row] = mean, rstd
        y = (x[row] - mean) * rstd * weight.astype(np.float32)
        if bias is not None:
            y = y + bias.astype(np.float32)
        out[row] = y
    return out, means, rstds


# ------------------------------------------------------------------------------------------------------------------
# rotary position embedding
# ------------------------------------------------------------------------------------------------------------------
def rotary_oracle(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Half-split convention: feature d < D/2 pairs with feature d + D/2.  out = x*cos + rotate_half(x)*sin in fp32;
    cos, sin broadcast against x ([.., S, D], both halves of the last dimension holding the same angles in the
    usual tables, though nothing here requires it).  Same rotation as experimental/llama-v2/llama/model.py:78-88 with
    the features permuted."""
    xf, c, s = x.float(), cos.float(), sin.float()
    half = x.shape[-1] // 2
    lo, hi = xf[..., :half], xf[..., half:]
    out_lo = lo * c[..., :half] - hi * s[..., :half]
    out_hi = hi * c[..., half:] + lo * s[..., half:]
    return torch.cat((out_lo, out_hi), dim=-1)


def rotary_complex_oracle(x: torch.Tensor, angles: torch.Tensor) -> torch.Tensor:
    """Interleaved-pair convention exactly as the reference computes it (experimental/llama-v2/llama/model.py:78-88):
    features (2i, 2i+1) are the real and imaginary parts of a complex number multiplied by exp(i*angle_i).
    x [.., S, D], angles [S, D/2]."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2).contiguous())
    rot = torch.polar(torch.ones_like(angles, dtype=torch.float32), angles.float())
    return torch.view_as_real(xc * rot).flatten(-2)


def e5m2_decode_oracle(raw: torch.Tensor) -> torch.Tensor:
    """fp8 e5m2 bytes (int8 / uint8) -> fp32, from the format's definition: 1 sign bit, 5 exponent bits (bias 15),
    2 mantissa bits; exponent 0 is subnormal (2^-14 · m/4), exponent 31 is inf (m = 0) or nan.  This is the storage of
    the reference's key/value caches (experimental/llama-v2/kernel/fused_kernel_fp8.py:40-56), which its attention kernel
    widens to fp16 before use (fused_kernel_attention.py:69-71).  Pinned in tests/test_oracle.py against
    torch.float8_e5m2 and against the fp16 encoding's upper byte.
    """
    b = raw.detach().cpu().view(torch.uint8).to(torch.int32)
    sign = torch.where((b >> 7) == 1, -1.0, 1.0)
    exp = (b >> 2) & 0x1F
    man = (b & 0x3).to(torch.float32)
    normal = torch.ldexp(1.0 + man / 4.0, exp - 15)
    subnormal = torch.ldexp(man / 4.0, torch.full_like(exp, -14))
    val = torch.where(exp == 0, subnormal, normal)
    val = torch.where(exp == 31, torch.where(man == 0, torch.tensor(float("inf")), torch.tensor(float("nan"))), val)
    return sign * val
