"""Oracle (test infrastructure): attention operators for causal_model built on the CPU oracle: lets a test run the
product's own module code with reference attention, on the CPU, to compare against the HIP run."""
import torch

from oracle import blocks, dense, monarch, prologue


class OracleOps:
    def __init__(self, compute_dtype=torch.float32):
        self.compute_dtype = compute_dtype
        self.calls = []

    def rope_table(self, head_dim, device):
        return None

    def qk_prologue(self, xq, xk, xv, wq, wk, num_heads, grid, start_frame, rope, k_cache, v_cache, start_idx,
                    f_tied=1, h_reduce=1, w_reduce=1, eps=1e-6):
        q, k, v = prologue.qk_prologue(xq, xk, xv, wq, wk, num_heads, grid, start_frame, eps)
        B, S, H, D = q.shape
        _, h, w = grid
        k_cache[:, start_idx:start_idx + S] = blocks.to_blocks(k, f_tied, h_reduce, w_reduce, h, w).reshape(B, S, H, D)
        v_cache[:, start_idx:start_idx + S] = blocks.to_blocks(v, f_tied, h_reduce, w_reduce, h, w).reshape(B, S, H, D)
        self.calls.append(("prologue", start_frame, start_idx, (f_tied, h_reduce, w_reduce)))
        return q

    def monarch_cached(self, q, k_view, v_view, f_tied, h_reduce, w_reduce, h, w, num_iters=1):
        B, _, H, D = q.shape
        qb = blocks.to_blocks(q, f_tied, h_reduce, w_reduce, h, w)
        b1, b2 = qb.shape[2], qb.shape[3]
        kb, vb = k_view.reshape(B, -1, b1, b2, H, D), v_view.reshape(B, -1, b1, b2, H, D)
        if num_iters == 1:
            out = monarch.monarch_1iter(qb, kb, vb, D ** -0.5, dtype=self.compute_dtype)
        else:
            out = monarch.monarch_iter(qb, kb, vb, D ** -0.5, num_iters, dtype=self.compute_dtype)
        self.calls.append(("monarch", k_view.shape[1]))
        return blocks.from_blocks(out, f_tied, h_reduce, w_reduce, h, w).to(q.dtype)

    def dense(self, q, k, v):
        self.calls.append(("dense", k.shape[1]))
        return dense.attention(q, k, v, dtype=self.compute_dtype).to(q.dtype)

    # element-wise operators of the block: the reference's eager chains (causal_model.py:1176-1205, model.py:462-478)
    def ln_modulate(self, x, scale, shift, eps):
        nf = scale.shape[1]
        n = torch.nn.functional.layer_norm(x, (x.shape[-1],), None, None, eps).type_as(x)
        return (n.unflatten(1, (nf, x.shape[1] // nf)) * (1 + scale) + shift).flatten(1, 2)

    def ln_affine(self, x, weight, bias, eps):
        return torch.nn.functional.layer_norm(x, (x.shape[-1],), weight, bias, eps).type_as(x)

    def gate_residual(self, x, y, gate=None):
        if gate is None:
            return x + y
        nf = gate.shape[1]
        return x + (y.unflatten(1, (nf, x.shape[1] // nf)) * gate).flatten(1, 2)

    def gate_residual_ln(self, x, y, gate, eps, scale=None, shift=None, weight=None, bias=None):
        x = self.gate_residual(x, y, gate)
        if weight is not None:
            return x, self.ln_affine(x, weight, bias, eps)
        return x, self.ln_modulate(x, scale, shift, eps)

    def linear(self, x, linear):
        return linear(x)

    def linear_gelu(self, x, linear):
        return torch.nn.functional.gelu(linear(x), approximate='tanh')

    def linear_gate_residual(self, x, h, linear, gate):
        return self.gate_residual(x, linear(h), gate)

    def rms_norm(self, x, weight, eps):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)).type_as(x) * weight
