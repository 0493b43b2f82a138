"""Decode steps replayed from captured HIP graphs: `DecodeSession` for one `SparseAttention` layer,
`TransformerDecodeSession` for the whole `Transformer`.

`SparseAttention.forward_inference` (NSA.py:338-547) derives every shape of a step on the host and
issues about a dozen launches; at small batch the host-side work is several times the kernels' run
time.  A `DecodeSession` owns fixed-capacity caches, keeps the token position and the number of
compressed keys in device memory (the kernels read them when they run, `nsa_decode_step_dyn`) and
records norm, projections, the attention step and the output projection into a HIP graph that is
replayed for every token.  Every `compress_block_sliding_stride` tokens a compression window is
complete (NSA.py:422-441); those steps replay a second graph that also gathers the window (rows
indexed from the device-side position), compresses it and appends the compressed key / value.

    out, cache = attn(prompt, return_cache=True)           # prefill, as in the reference
    session = DecodeSession(attn, cache, max_len=65536)
    for x in tokens:                                         # x: 'b 1 dim'
        y = session.step(x)
    cache = session.cache()                                  # back to the module's cache format

The reference has no counterpart; results equal `forward_inference` up to the order in which split
partial results are merged (the split is sized for the capacity rather than the current length).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from .ops import _kernel_dim, _pad_dim

_BF16 = torch.bfloat16


def ring_rows(first, count_range: torch.Tensor, ring: int) -> torch.Tensor:
    """Rows of a position-indexed ring (position p lives in row p % ring) that hold positions first, first+1, ...:
    `first` is an int or a 0-dim integer tensor (e.g. a device-side counter), `count_range` = arange(count).  Positions
    before the sequence start map to rows that have not been written yet (ring >= count), i.e. to zeros."""
    return torch.remainder(first + count_range, ring)


class DecodeSession:
    def __init__(self, module, cache, max_len: int, capture: bool = True):
        m = self.module = module
        assert m.causal, 'inference only relevant for autoregressive'
        (cache_k, cache_v), ((cache_ck, cache_cv), (run_k, run_v)) = cache
        if not cache_k.is_cuda:
            raise RuntimeError("DecodeSession runs on the GPU only (HIP kernels, no CPU fallback)")
        if m.to_qkv.weight.dtype != _BF16:
            raise NotImplementedError("DecodeSession needs a bf16 module (the raw key / value window is kept in bf16)")
        dev = cache_k.device
        b, hk, t, _ = cache_k.shape
        d0 = m.dim_head
        # the kernels hold 64 or 128 features per head: any other head dimension lives zero-padded in the session's
        # buffers (zero features change neither logits nor outputs; the softmax scale stays that of d0), and the
        # projection weights are copied with zero rows / columns so that the GEMMs read and write the padded layout
        d = _kernel_dim(d0)
        self.d0 = d0
        st, cbs = m.compress_block_sliding_stride, m.compress_block_size
        nc = cache_ck.shape[-2]
        if max_len <= t:
            raise ValueError(f"max_len {max_len} leaves no room after the {t} cached tokens")
        self.b, self.hk, self.hq, self.d = b, hk, m.heads, d
        self.st, self.cbs, self.max_len = st, cbs, int(max_len)
        self.pos, self.nc = t, nc                                   # host mirrors of the device state
        self.max_nc = (max(self.max_len // st, nc, 1) + 7) // 8 * 8        # rows of 16-byte-aligned fp32 logits

        def grown(src, rows):
            buf = torch.zeros((b, hk, rows, d), dtype=_BF16, device=dev)
            buf[:, :, :src.shape[-2], :src.shape[-1]].copy_(src)      # the module's own decode steps hand back padded rows
            return buf
        self.K, self.V = grown(cache_k, self.max_len), grown(cache_v, self.max_len)
        # one spare row: the capture warm-up and the recording of the window-completing graph write row `nc` of the compressed
        # caches whatever nc is, also when the prefill already filled all max_nc rows (the real steps never do: completes_window)
        self.CK, self.CV = grown(cache_ck, self.max_nc + 1), grown(cache_cv, self.max_nc + 1)

        # raw (un-rotated) keys / values of the last tokens, position p in row p % ring; rows never written are zero, which is
        # also what the window of the first compression steps holds for positions before the sequence start (NSA.py:866)
        self.ring = R = 2 * cbs
        self.ring_k = torch.zeros((b, hk, R, d), dtype=_BF16, device=dev)
        self.ring_v = torch.zeros((b, hk, R, d), dtype=_BF16, device=dev)
        lr = run_k.shape[-2]
        if lr > R:
            raise ValueError("the cache's open compression window is longer than two compression blocks")
        if lr:
            rows = ring_rows(t - lr, torch.arange(lr, device=dev), R)
            self.ring_k[:, :, rows] = _pad_dim(run_k.to(_BF16), d)
            self.ring_v[:, :, rows] = _pad_dim(run_v.to(_BF16), d)
        self._ar = torch.arange(cbs, device=dev, dtype=torch.int32)
        self.state = torch.tensor([t, nc], dtype=torch.int32, device=dev)
        self.mem_k = _pad_dim(m.compress_mem_kv[0].detach().to(_BF16), d).contiguous()
        self.mem_v = _pad_dim(m.compress_mem_kv[1].detach().to(_BF16), d).contiguous()
        self.freqs = _pad_dim(m.rotary_emb.freqs.detach().to(torch.float32), d // 2).contiguous()   # frequency 0: no rotation

        def padded_heads(w, dim):            # 'heads * d0' along `dim` of a weight -> 'heads * d' with zeros
            if d == d0:
                return w
            shape = list(w.shape)
            shape[dim:dim + 1] = [shape[dim] // d0, d0]
            w = _pad_dim(w.reshape(shape).movedim(dim + 1, -1), d).movedim(-1, dim + 1)
            shape[dim:dim + 2] = [shape[dim] * d]
            return w.reshape(shape)
        w_qkv = padded_heads(m.to_qkv.weight.detach(), 0)
        self.w_out = padded_heads(m.combine_heads.weight.detach(), 1).contiguous() if d != d0 else None

        # q, k, v and the strategy-gate logits come out of one GEMM: the gate projection's rows are appended to the qkv
        # weight (a copy: the session does not follow later changes of the module's parameters), its bias is added where the
        # logits are used
        gate = m.to_strategy_combine[0]
        self.fused_gate = isinstance(gate, torch.nn.Linear) and gate.in_features == m.to_qkv.in_features and gate.out_features == 3 * m.heads
        if self.fused_gate:
            pad = -3 * m.heads % 8                                  # rows of the GEMM output stay 16-byte aligned
            self.w_cat = torch.cat((w_qkv, gate.weight.detach().to(_BF16),
                                    torch.zeros((pad, m.to_qkv.in_features), dtype=_BF16, device=dev)), dim=0).contiguous()
            self.gate_bias = gate.bias.detach().to(_BF16).contiguous() if gate.bias is not None else None
        else:                                                       # a caller-supplied strategy network runs as it is
            self.w_cat, self.gate_bias = w_qkv.contiguous(), None
        self.x_buf = torch.zeros((b, 1, m.to_qkv.in_features), dtype=_BF16, device=dev)
        self._desc, self._ws = self._make_desc(dev)
        self.graphs = None
        if capture:
            # the libraries initialise themselves on first use (outside the capture); the warm-up steps write row `pos` of
            # the caches and row `nc` of the compressed caches, which the first real steps overwrite, and leave both counters alone
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side), torch.no_grad():
                for _ in range(2):
                    self.layer_step(self.x_buf, advance=0)
                    self.compress_window(count=False)
            torch.cuda.current_stream(dev).wait_stream(side)
            self.graphs, self.outs = [], []
            for event in (False, True):                             # [0]: ordinary step, [1]: step that completes a window
                g = torch.cuda.CUDAGraph()
                with torch.no_grad(), torch.cuda.graph(g):
                    out = self.layer_step(self.x_buf, advance=1)
                    if event:
                        self.compress_window()
                self.graphs.append(g)
                self.outs.append(out)

    # ---------------------------------------------------------------------------------------

    def _make_desc(self, dev):
        m = self.module
        dsc = _lib.DecodeStepDesc()
        dsc.batch, dsc.heads, dsc.kv_heads, dsc.dim_head = self.b, self.hq, self.hk, self.d
        dsc.pos, dsc.num_compressed = self.max_len - 1, self.max_nc
        dsc.per_block, dsc.block = m.selection_block_size // self.st, m.selection_block_size
        dsc.num_sel, dsc.share = m.num_selected_blocks, int(bool(m.query_heads_share_selected_kv))
        dsc.window, dsc.scale = m.sliding_window_size, self.d0 ** -0.5
        dsc.num_mem = self.mem_k.shape[-2]
        dsc.kc_stride[:] = self.K.stride()[:3]
        dsc.vc_stride[:] = self.V.stride()[:3]
        dsc.ck_stride[:] = self.CK.stride()[:3]
        dsc.cv_stride[:] = self.CV.stride()[:3]
        dsc.krun_stride[:] = self.ring_k.stride()[:2]
        dsc.vrun_stride[:] = self.ring_v.stride()[:2]
        # q / k / v are views of the qkv projection's output: 'b 1 (h d)' -> strides {row, head}
        width = self.w_cat.shape[0]
        for name in ("q_stride", "k_stride", "v_stride"):
            getattr(dsc, name)[:] = (width, self.d)
        nbytes = C.c_size_t()
        _lib.check(_lib.lib().nsa_decode_step_workspace_bytes(C.byref(dsc), C.byref(nbytes), None, None, None),
                   "nsa_decode_step_workspace_bytes")
        return dsc, torch.empty(nbytes.value, dtype=torch.uint8, device=dev)

    def layer_step(self, x_in: torch.Tensor, advance: int):
        """The layer's decode step on `x_in` 'b 1 dim' as a sequence of launches with no host-side dependence on the
        position (recordable into a graph); advance != 0 increments the device-side position afterwards."""
        m = self.module
        x = m.norm(x_in)
        qkvg = torch.nn.functional.linear(x, self.w_cat)             # 'b 1 ((hq + 2 hk) d + 3 hq)', contiguous
        hq, hk, d = self.hq, self.hk, self.d
        merged = torch.empty((self.b, 1, hq * d), dtype=_BF16, device=x.device)
        p = qkvg.data_ptr()
        if self.fused_gate:
            gate_ptr, gate_row = p + 2 * (hq + 2 * hk) * d, qkvg.shape[-1]
        else:
            gl = m.to_strategy_combine[0](x).to(_BF16).contiguous()
            gate_ptr, gate_row = gl.data_ptr(), 0
        _lib.check(_lib.lib().nsa_decode_step_dyn(
            C.byref(self._desc), self.state.data_ptr(), p, p + 2 * hq * d, p + 2 * (hq + hk) * d, self.freqs.data_ptr(),
            self.K.data_ptr(), self.V.data_ptr(), self.CK.data_ptr(), self.CV.data_ptr(), self.mem_k.data_ptr(), self.mem_v.data_ptr(),
            self.ring_k.data_ptr(), self.ring_v.data_ptr(), self.ring_k.stride(2), self.ring_v.stride(2), self.ring,
            gate_ptr, gate_row, self.gate_bias.data_ptr() if self.gate_bias is not None else None,
            self._ws.data_ptr(), self._ws.numel(), merged.data_ptr(), int(advance),
            torch.cuda.current_stream(x.device).cuda_stream), "nsa_decode_step_dyn")
        if self.w_out is not None:
            return torch.nn.functional.linear(merged, self.w_out, m.combine_heads.bias)
        return m.combine_heads(merged)

    def compress_window(self, count: bool = True):
        """Compress the window that ends at the device-side position (already advanced past the newest token) and append it
        to the compressed caches (NSA.py:422-441); every index comes from device memory."""
        m = self.module
        rows = ring_rows(self.state[0] - self.cbs, self._ar, self.ring)
        wk = self.ring_k.index_select(2, rows)[..., :self.d0]
        wv = self.ring_v.index_select(2, rows)[..., :self.d0]
        at = self.state[1:2].long().clamp(max=self.CK.shape[2] - 1)    # the spare last row at most, whatever the counter holds
        self.CK.index_copy_(2, at, _pad_dim(m.k_compress((wk + m.k_intrablock_positions)[:, :, None]).to(_BF16), self.d))
        self.CV.index_copy_(2, at, _pad_dim(m.v_compress((wv + m.v_intrablock_positions)[:, :, None]).to(_BF16), self.d))
        if count:
            self.state[1:2].add_(1)

    def completes_window(self) -> bool:
        """Whether the token at the current position completes a compression window."""
        return (self.pos + 1) % self.st == 0 and self.nc < self.max_nc

    def advance_host(self, event: bool):
        """Follow on the host what a replayed step did to the device-side counters."""
        self.pos += 1
        self.nc += int(event)

    @torch.no_grad()
    def step(self, x: torch.Tensor) -> torch.Tensor:
        """x 'b 1 dim': the token at position `self.pos`.  Returns the layer output 'b 1 dim' (a new tensor)."""
        if self.graphs is None:
            raise RuntimeError("DecodeSession was built with capture=False (its launches belong to an enclosing graph)")
        if self.pos >= self.max_len:
            raise RuntimeError(f"DecodeSession: capacity of {self.max_len} tokens reached")
        event = self.completes_window()
        self.x_buf.copy_(x)
        self.graphs[event].replay()
        self.advance_host(event)
        return self.outs[event].clone()

    def cache(self):
        """The caches in the module's format `((k, v), ((ck, cv), (run_k, run_v)))` (copies of the filled parts)."""
        t, st, cbs = self.pos, self.st, self.cbs
        first = (t // st) * st - (cbs - st)                          # first position of the open window
        rows = ring_rows(first, torch.arange(t - first, device=self.K.device), self.ring)
        d0 = self.d0        # as the module's own decode step keeps them: keys / values and window rows padded, compressed keys not
        run_k, run_v = self.ring_k.index_select(2, rows), self.ring_v.index_select(2, rows)
        if first < 0:                                                # positions before the sequence start read as zero
            run_k[:, :, :-first] = 0
            run_v[:, :, :-first] = 0
        return ((self.K[:, :, :t].clone(), self.V[:, :, :t].clone()),
                ((self.CK[:, :, :self.nc, :d0].clone(), self.CV[:, :, :self.nc, :d0].clone()), (run_k, run_v)))


class TransformerDecodeSession:
    """Token-by-token decoding of a `Transformer` (transformer.py:213-252 with use_cache_kv) as one graph replay per
    token: embedding, every layer's attention step and feed-forward, final norm and logits.  `caches` is what
    `model(prompt, return_cache=True)` returned; `max_len` the longest sequence to decode to."""

    def __init__(self, model, caches, max_len: int):
        self.model = model
        dev = caches[0][0][0].device
        b = caches[0][0][0].shape[0]
        self.layers = [DecodeSession(attn, cache, max_len, capture=False) for (attn, _), cache in zip(model.layers, caches)]
        self.tok = torch.zeros((b, 1), dtype=torch.long, device=dev)
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(2):
                self._body(advance=0, event=True, count=False)
        torch.cuda.current_stream(dev).wait_stream(side)
        self.graphs, self.outs = [], []
        for event in (False, True):
            g = torch.cuda.CUDAGraph()
            with torch.no_grad(), torch.cuda.graph(g):
                out = self._body(advance=1, event=event, count=True)
            self.graphs.append(g)
            self.outs.append(out)

    def _body(self, advance: int, event: bool, count: bool):
        model = self.model
        x = model.token_emb(self.tok)
        for sess, (_, ff) in zip(self.layers, model.layers):
            a = sess.layer_step(x, advance)
            if event:
                sess.compress_window(count)
            x = a + x
            x = ff(x) + x
        return model.to_logits(model.norm(x))

    @property
    def pos(self) -> int:
        return self.layers[0].pos

    @torch.no_grad()
    def step(self, token: torch.Tensor) -> torch.Tensor:
        """token 'b' or 'b 1' (int64): the token at the current position.  Returns the logits 'b 1 vocab' for the next one."""
        first = self.layers[0]
        if first.pos >= first.max_len:
            raise RuntimeError(f"TransformerDecodeSession: capacity of {first.max_len} tokens reached")
        event = first.completes_window()
        self.tok.copy_(token.reshape(self.tok.shape))
        self.graphs[event].replay()
        for sess in self.layers:
            sess.advance_host(event)
        return self.outs[event].clone()
