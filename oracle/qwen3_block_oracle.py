"""CPU restatement of the per-head q/k RMSNorm and rotary embedding of the reference's Qwen3
attention block (the parity oracle for the fused norm + rotation + cache-write kernel).

TEST INFRASTRUCTURE ONLY.  Nothing under the product package imports this module; only tests/
do, as the checker.  It follows the reference's module code:

  rms_norm            src/distributed/tensor_parallel.py:78-84    x.float(), mean of squares, rsqrt, weight * x, cast back
  inv_freq            src/distributed/tensor_parallel.py:389-395  1 / theta ** (arange(0, D, 2) / D)
  apply_rotary_emb    src/distributed/tensor_parallel.py:397-419  cos / sin of outer(pos, inv_freq) repeated over both
                                                                  halves; x * cos + cat(-x2, x1) * sin
  qk_norm_rope        src/distributed/tensor_parallel.py:453-464  norm of q and k, then rotation of both
  add_rms_norm        src/distributed/tensor_parallel.py:640-651  residual + x in the activation dtype, then rms_norm of it
  swiglu              src/distributed/tensor_parallel.py:295-299  F.silu(gate) * up

The reference's rotation multiplies a 16-bit activation by fp32 cos / sin and therefore returns
fp32; the block that consumes it casts back to the activation dtype before attention
(:473-476), which `apply_rotary_emb(..., cast_back=True)` does here.

Pinning (tests/test_oracle_qwen3_block.py), none of which retypes a formula:
  * rms_norm: with weight 1 every output row has mean square 1 (up to eps); scaling the input by
    a constant leaves the output unchanged; a one-hot row of height a gives sqrt(D) * sign(a).
  * apply_rotary_emb: position 0 is the identity; each pair (x[i], x[i + D/2]) keeps its
    Euclidean length; rotating by m then reading the scores against a key rotated by n depends
    on m - n only (the property the embedding exists for); pair i at position p has turned by
    exactly p * theta^(-2i/D) radians (checked with atan2 in fp64).
  * qk_norm_rope: equals the two steps applied one after the other.
  * add_rms_norm: the sum is the correctly rounded sum (checked in fp64); the normed output is
    rms_norm of that sum.
  * swiglu: silu(0) = 0, silu(x) -> x for large x and -> 0 for large -x, silu(x) - silu(-x) = x
    (all in fp64 to rounding), and against x * sigmoid(x) evaluated in fp64.
"""
import torch


def rms_norm(x, weight, eps=1e-6):
    input_dtype = x.dtype
    xf = x.float()
    variance = xf.pow(2).mean(-1, keepdim=True)
    xf = xf * torch.rsqrt(variance + eps)
    return (weight * xf).to(input_dtype)


def inv_freq(head_dim, theta=1000000.0):
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))


def apply_rotary_emb(x, positions, inv_f, cast_back=True):
    """x [T, H, D], positions [T]."""
    half = x.shape[-1] // 2
    freqs = torch.outer(positions.float(), inv_f)
    emb = torch.cat([freqs, freqs], dim=-1)
    cos = emb.cos().unsqueeze(1)
    sin = emb.sin().unsqueeze(1)
    x1 = x[..., :half]
    x2 = x[..., half:]
    rotated = torch.cat([-x2, x1], dim=-1)
    out = x * cos + rotated * sin
    return out.to(x.dtype) if cast_back else out


def qk_norm_rope(q, k, q_weight, k_weight, eps, positions, inv_f):
    q = apply_rotary_emb(rms_norm(q, q_weight, eps), positions, inv_f)
    k = apply_rotary_emb(rms_norm(k, k_weight, eps), positions, inv_f)
    return q, k


def add_rms_norm(x, delta, weight, eps=1e-6):
    """(residual + x, norm of it): the block's add is done in the activation dtype, the norm
    sees the rounded sum."""
    total = x + delta
    return total, rms_norm(total, weight, eps)


def swiglu(gate, up):
    import torch.nn.functional as F
    return F.silu(gate) * up
