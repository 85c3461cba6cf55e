"""fp32 CPU evaluation of single rows and weight-gradient blocks of the MoE expert layer.  Test infrastructure.

Used by the full-size GPU parity tests, where running the whole-layer oracle would take minutes; pinned on the CPU
against the oracle's own autograd on a small configuration (tests/test_oracle_pins.py)."""
import torch

BF = torch.bfloat16


def r16(t):
    """Round an fp32 tensor to bf16 and back: the rounding every op's bf16 output goes through."""
    return t.to(BF).float()


class RowRef:
    """fp32 CPU evaluation of single rows of the layer (a row = one (token, slot) pair in expert-major order)."""

    def __init__(self, cfg, x, p, idx, w1, w2, gy):
        self.cfg = cfg
        self.r = r16 if x.dtype == BF else (lambda t: t)       # fp32 inputs: nothing is rounded
        self.K, self.F, self.E = cfg["K"], cfg["F"], cfg["E"]
        self.x, self.p, self.gy = x.cpu().float(), p.cpu().float(), gy.cpu().float()
        self.idx = idx.cpu()
        self.w1, self.w2 = w1, w2                      # device tensors; slices are fetched when needed
        flat = self.idx.reshape(-1)
        self.fwd = torch.sort(flat.float(), stable=True)[1]            # flat position of row r
        self.rmap = torch.empty_like(self.fwd)
        self.rmap[self.fwd] = torch.arange(self.fwd.numel())
        self.expert_of_row = flat[self.fwd]
        self.counts = torch.bincount(flat, minlength=self.E)
        self.offsets = torch.cat([torch.zeros(1, dtype=torch.long), torch.cumsum(self.counts, 0)])
        self._w = {}

    def weights(self, e):
        if e not in self._w:
            self._w = {e: (self.w1[e].cpu().float(), self.w2[e].cpu().float())}    # keep one expert at a time
        return self._w[e]

    def rows_of_token(self, t):
        return [int(self.rmap[t * self.K + j]) for j in range(self.K)]

    def eval_rows(self, rows):
        """For the given rows (any experts): dict row -> (o, dperm) with o the row's second-matmul output and
        dperm the gradient that flows back to the permuted input row."""
        out = {}
        rows = sorted(set(rows), key=lambda r: int(self.expert_of_row[r]))
        by_expert = {}
        for r in rows:
            by_expert.setdefault(int(self.expert_of_row[r]), []).append(r)
        F = self.F
        for e, rs in by_expert.items():
            w1, w2 = self.weights(e)
            pos = self.fwd[rs]
            tok, slot = pos // self.K, pos % self.K
            xr = self.x[tok]
            pr = self.p[tok, slot].unsqueeze(1)
            h = self.r(xr @ w1)
            gate, up = h[:, :F], h[:, F:]
            sig = torch.sigmoid(gate)
            act = self.r(gate * sig * up)
            o = self.r(act @ w2)
            g_o = self.r(pr * self.gy[tok])                       # unpermute backward: rows of dY scaled by prob
            dact = self.r(g_o @ w2.t())
            dh = self.r(torch.cat([dact * up * (sig * (1 + gate * (1 - sig))), dact * gate * sig], dim=1))
            dperm = self.r(dh @ w1.t())
            for i, r in enumerate(rs):
                out[r] = (o[i], dperm[i])
        return out

    def token_refs(self, tokens):
        """Expected layer output, dX and grad_probs of the given tokens."""
        rows = [r for t in tokens for r in self.rows_of_token(t)]
        ev = self.eval_rows(rows)
        outs, dxs, dps = [], [], []
        for t in tokens:
            rs = self.rows_of_token(t)
            outs.append(sum(self.p[t, j] * ev[r][0] for j, r in enumerate(rs)))
            dxs.append(sum(ev[r][1] for r in rs))
            dps.append(torch.stack([torch.dot(self.gy[t], ev[r][0]) for r in rs]))
        return torch.stack(outs), torch.stack(dxs), torch.stack(dps)

    def dw_blocks(self, e, ks, fs, hs):
        """Blocks of expert e's weight gradients: dW1[e][ks, fs] (gate columns), dW1[e][ks, F + fs] (up columns)
        and dW2[e][fs, hs], with ks / fs / hs index tensors."""
        F = self.F
        r0, r1 = int(self.offsets[e]), int(self.offsets[e + 1])
        pos = self.fwd[r0:r1]
        tok, slot = pos // self.K, pos % self.K
        xe = self.x[tok]                                                   # [rows, H]
        g_o = self.r(self.p[tok, slot].unsqueeze(1) * self.gy[tok])           # [rows, H]
        cols = torch.cat([fs, F + fs]).to(self.w1.device)
        w1c = self.w1[e][:, cols].cpu().float()                            # [H, 2*|fs|]
        w2r = self.w2[e][fs.to(self.w2.device), :].cpu().float()           # [|fs|, H]
        h = self.r(xe @ w1c)
        gate, up = h[:, :len(fs)], h[:, len(fs):]
        sig = torch.sigmoid(gate)
        act = self.r(gate * sig * up)
        dact = self.r(g_o @ w2r.t())
        dgate = self.r(dact * up * (sig * (1 + gate * (1 - sig))))
        dup = self.r(dact * gate * sig)
        xk = xe[:, ks]
        return xk.t() @ dgate, xk.t() @ dup, act.t() @ g_o[:, hs]


