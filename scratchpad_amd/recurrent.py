"""Recurrent token mixer with a per-head matrix state (RWKV-style time mixing) over the HIP kernels of csrc/wkv.hip.

Per token t with layer input h[t] (the fp32 residual stream) and h[t-1] (zeros at a sequence's first token):
  m_s = h[t] + (h[t-1] - h[t]) * mu_s                      one mix per projection s in (r, k, v, g, w)
  r, k, v = W_r m_r, W_k m_k, W_v m_v   gate = silu(W_g m_g)   decay = exp(-exp(W_w2 tanh(W_w1 m_w) + w0))
  o = (S + diag(u) k v^T)^T r ;  S <- diag(decay) S + k v^T     per head, S in fp32 in the RecurrentStatePool
  out = W_o ((o / rms_head(o)) * norm * gate)
The four projections that feed the recurrence run as ONE batched matrix product over their stacked weights."""
import torch
from torch import nn

from . import _native
from .forward_info import ForwardBatch


class WKVMixer(nn.Module):
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, width: int, heads: int, dim: int, decay_rank: int, layer_id: int, eps: float, dtype=None):
        super().__init__()
        self.width, self.heads, self.dim, self.layer_id, self.eps = width, heads, dim, layer_id, eps
        n = heads * dim
        f32 = dict(dtype=torch.float32)
        self.mu = nn.Parameter(torch.zeros(len(self.MIXES), width, **f32), requires_grad=False)
        self.rkvg = nn.Parameter(torch.empty(4, n, width, dtype=dtype), requires_grad=False)
        self.w1 = nn.Parameter(torch.empty(decay_rank, width, dtype=dtype), requires_grad=False)
        self.w2t = nn.Parameter(torch.zeros(decay_rank, n, **f32), requires_grad=False)      # W_w2 transposed, fp32
        self.w0 = nn.Parameter(torch.zeros(n, **f32), requires_grad=False)
        self.u = nn.Parameter(torch.zeros(heads, dim, **f32), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(n, **f32), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, n, dtype=dtype), requires_grad=False)

    def forward(self, x: torch.Tensor, forward_batch: ForwardBatch) -> torch.Tensor:
        """x: the fp32 stream [T, W] -> the mixer's output [T, W] in the projections' dtype"""
        seq = forward_batch.attn_backend.seq
        states = forward_batch.state_pool
        dtype = self.o.dtype
        shift = states.shift_state(self.layer_id)
        mixes = _native.token_shift(x, self.mu.data, shift, seq, dtype)               # [5, T, W]
        _native.save_last_rows(shift, x, seq)                                         # after its only reader this step
        rkvg = torch.bmm(mixes[:4], self.rkvg.transpose(1, 2))                        # [4, T, H * D]
        decay = _native.wkv_decay(_native.linear(mixes[4], self.w1), self.w2t.data, self.w0.data)
        o = _native.wkv_recurrence(rkvg[0], rkvg[1], rkvg[2], rkvg[3], decay, self.u.data, self.norm.data,
                                   states.matrix_state(self.layer_id), seq, self.heads, self.dim, self.eps)
        return _native.linear(o, self.o)
