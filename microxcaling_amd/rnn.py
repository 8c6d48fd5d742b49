"""MX LSTM: torch.nn.LSTM's parameters and interface with every matmul, gate activation and
elementwise step done by the MX ops, like the reference's mx/rnn.py.  Sequence-first tensors or
PackedSequence inputs; no projection (proj_size = 0)."""
import torch
from torch.nn.utils.rnn import PackedSequence

from .activations import sigmoid, tanh
from .linear import linear
from .simd_ops import simd_add, simd_mul
from .specs import apply_mx_specs, mx_assert_test


def _cut(state, start, end):
    """Columns start:end (batch entries) of an (h, c) pair shaped (1, N, H)."""
    return (state[0][:, start:end], state[1][:, start:end])


def _join(states, dim):
    return (torch.cat([s[0] for s in states], dim=dim), torch.cat([s[1] for s in states], dim=dim))


class LSTM(torch.nn.LSTM):
    """Layer l, direction d uses weight_ih_l{l}{_reverse}, weight_hh_..., bias_...; gates are
    ordered input, forget, cell, output as in torch (mx/rnn.py:20-362)."""

    def __init__(self, *args, mx_specs=None, name='', **kwargs):
        super().__init__(*args, **kwargs)
        assert self.batch_first == False
        assert self.proj_size == 0
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)
        self.name = name
        self.dropout_layer = torch.nn.Dropout(p=self.dropout)

    # ---- one direction of one layer ---------------------------------------------------------
    def _params(self, kind, layer, reverse):
        suffix = '%s_l%d%s' % (kind, layer, '_reverse' if reverse else '')
        return getattr(self, 'weight_' + suffix), getattr(self, 'bias_' + suffix, None)

    def _project_inputs(self, x, layer, reverse):
        """The input half of the gate pre-activations for every time step at once."""
        w, b = self._params('ih', layer, reverse)
        return linear(x, w, bias=b, mx_specs=self.mx_specs,
                      name=self.name + ('.InputReverseLinear' if reverse else '.InputLinear'))

    def _cell(self, xw, state, layer, reverse=False):
        """One time step from the pre-projected input xw and the (h, c) state."""
        s = self.mx_specs
        w, b = self._params('hh', layer, reverse)
        h, c = state
        gates = simd_add(xw, linear(h, w, bias=b, mx_specs=s, name=self.name + '.HiddenLinear'), mx_specs=s)
        gi, gf, gg, go = gates.chunk(4, dim=-1)
        i = sigmoid(gi, mx_specs=s)
        f = sigmoid(gf, mx_specs=s)
        g = tanh(gg, mx_specs=s)
        o = sigmoid(go, mx_specs=s)
        c = simd_add(simd_mul(f, c, mx_specs=s), simd_mul(i, g, mx_specs=s), mx_specs=s)
        h = simd_mul(o, tanh(c, mx_specs=s), mx_specs=s)
        return h, c

    # ---- packed sequences: the batch shrinks as shorter sequences end ---------------------------
    def _run_packed(self, state, xw, batch_sizes, layer):
        finished, outputs = [], []
        offset, live = 0, batch_sizes[0]
        for n in batch_sizes:
            step = xw[offset:offset + n]
            offset += n
            if live > n:                       # sequences that just ended keep their last state
                finished.append(_cut(state, n, live))
                state = _cut(state, 0, n)
            live = n
            state = self._cell(step, state, layer, reverse=False)
            outputs.append(state[0])
        finished.append(state)
        finished.reverse()
        return _join(finished, dim=1), torch.cat(outputs, dim=1).squeeze(0)

    def _run_packed_reverse(self, state0, xw, batch_sizes, layer):
        offset, live = len(xw), batch_sizes[-1]
        state = _cut(state0, 0, live)
        outputs = []
        for n in reversed(batch_sizes):
            if n > live:                       # sequences that start here join with their initial state
                state = _join([state, _cut(state0, live, n)], dim=1)
            step = xw[offset - n:offset]
            offset -= n
            live = n
            state = self._cell(step, state, layer, reverse=True)
            outputs.append(state[0])
        outputs.reverse()
        return state, torch.cat(outputs, dim=1).squeeze(0)

    def forward(self, input, hx=None):
        if self.mx_none:
            return super().forward(input, hx)
        packed = isinstance(input, PackedSequence)
        if packed:
            data, batch_sizes, sorted_indices, unsorted_indices = input
            max_batch = int(batch_sizes[0])
        else:
            data, batch_sizes, sorted_indices, unsorted_indices = input, None, None, None
            max_batch = input.size(0) if self.batch_first else input.size(1)
        D = 2 if self.bidirectional else 1
        if hx is None:
            zeros = lambda: torch.zeros(self.num_layers * D, max_batch, self.hidden_size,
                                        dtype=data.dtype, device=data.device)
            hx = (zeros(), zeros())
        else:
            hx = self.permute_hidden(hx, sorted_indices)
        self.check_forward_args(data, hx, batch_sizes)
        hs, cs = hx
        assert hs.shape[0] == D * self.num_layers and cs.shape[0] == D * self.num_layers
        hs, cs = hs.unsqueeze(1).unbind(0), cs.unsqueeze(1).unbind(0)      # per (layer, direction): (1, N, H)

        final_h, final_c = [], []
        seq = data
        for l in range(self.num_layers):
            fwd = (hs[D * l], cs[D * l])
            xw = self._project_inputs(seq, l, reverse=False)
            if self.bidirectional:
                bwd = (hs[D * l + 1], cs[D * l + 1])
                xw_r = self._project_inputs(seq, l, reverse=True)
            if packed:
                sizes = [int(b) for b in batch_sizes]
                fwd, out = self._run_packed(fwd, xw, sizes, l)
                if self.bidirectional:
                    bwd, out_r = self._run_packed_reverse(bwd, xw_r, sizes, l)
            else:
                steps, steps_r = [], []
                for t in range(data.shape[0]):
                    fwd = self._cell(xw[t], fwd, l, reverse=False)
                    steps.append(fwd[0])
                    if self.bidirectional:
                        bwd = self._cell(xw_r[-1 - t], bwd, l, reverse=True)
                        steps_r.insert(0, bwd[0])
                out = torch.cat(steps, dim=0)
                if self.bidirectional:
                    out_r = torch.cat(steps_r, dim=0)
            if self.bidirectional:
                final_h.append(torch.cat((fwd[0], bwd[0]), dim=0))
                final_c.append(torch.cat((fwd[1], bwd[1]), dim=0))
                assert len(out) == len(out_r)
                seq = torch.cat((out, out_r), dim=-1)
            else:
                final_h.append(fwd[0])
                final_c.append(fwd[1])
                seq = out
            if l != self.num_layers - 1 and self.dropout > 0:
                seq = self.dropout_layer(seq)

        hidden = self.permute_hidden((torch.cat(final_h, dim=0), torch.cat(final_c, dim=0)), unsorted_indices)
        if packed:
            return PackedSequence(seq, batch_sizes, sorted_indices, unsorted_indices), hidden
        return seq, hidden
