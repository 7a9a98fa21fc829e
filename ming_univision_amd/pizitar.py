"""Pizitar: a decoder-only language model of latent-attention layers, served by libmingnative's latent-cache step function
(mingnative.h section 9: mn_seq_step).

Per layer, with x the fp32 residual stream of a token:
    n  = LN(x)                                  weight + bias
    h  = n + F(n)                               F: causal per-channel filter over the last `taps` inputs of the sequence
    y  = mixer(h)                               latent attention: only c = RMSnorm(W_dkv h) is cached per token; keys and values of
                                                every head are W_uk c and W_uv c, so the scores are (W_uk^T q) . c and the heads'
                                                outputs W_uv (sum_j p_j c_j) — attention runs against the latents themselves
    x += LN(sigmoid(W_g1 n + b_g1) * y)
    x += LN(sigmoid(W_g2 n2 + b_g2) * W_down P(W_up n2)),  n2 = LN(x),  P = a U(z) + b U(z^2) + c U(z^3) + e,  U(v) = v / rms(v)
then LN, the vocabulary projection and a tanh soft cap.  A layer may attend another layer's latents (`kv_from`).

This module owns HBM residency, like bailing_moe.py for the other decoder:
  * weights bf16; the projections that read the same rows are stacked at load ([q-latent ; kv-latent], [q ; gate ; kv-latent],
    [feed-forward gate ; up]) and W_uk is stored per head transposed, so absorb and expand are plain batched products;
  * one fp32 latent arena [n_seq, t_max, kv_rank] per layer that projects latents, one fp32 filter state
    [layers, n_seq, taps - 1, width]; cache sequences are numbered as in the other decoder (`sequences.SequenceSlots`);
  * per-row int32 bookkeeping on the device, so a lock-step decode loop never syncs with the host.
`arith`: "bf16" = matrix products of steps above 8 rows on the bf16 MFMA kernels (fp32 accumulate), everything else fp32;
"f32" = fp32 FMA everywhere.
"""
import ctypes as C
import glob
import os

import numpy as np
import torch

from . import _lib, ops
from ._lib import SeqLayer, SeqModel, SeqState, check, current_stream, lib, ptr
from .configuration import PizitarConfig, pizitar_param_shapes
from .sequences import SequenceSlots, rows_of_spans

MAX_ROWS = 2048          # rows of one pass through the stack; longer inputs run as several passes
ARITH = {"bf16": 0, "f32": 1}


class PizitarDecoder:
    """Weights + latent arenas + filter states + the C-ABI tables of the stack."""

    def __init__(self, cfg: PizitarConfig, sd, t_max=2048, n_seq=1, arith="bf16"):
        """sd: {checkpoint tensor name: bf16 CUDA tensor}."""
        assert arith in ARITH, f"arith={arith!r}: 'bf16' or 'f32'"
        self.cfg, self.arith = cfg, arith
        missing = [k for k, shp in pizitar_param_shapes(cfg).items() if k not in sd or tuple(sd[k].shape) != tuple(shp)]
        if missing:
            raise ValueError(f"checkpoint does not fit the configuration: missing or mis-shaped tensors {missing[:8]}")
        dev = sd["embed"].device
        self.device = dev
        self.embed_w, self.head_w = sd["embed"].contiguous(), sd["head"].contiguous()
        self.t_max, self.n_seq = int(t_max), int(n_seq)
        W = cfg.width
        self._keep = []                                  # packed tensors the C tables point to
        self.arena_of, ranks = {}, []
        layers = (SeqLayer * len(cfg.layers))()
        for i, ly in enumerate(cfg.layers):
            m, mlp, p, L = ly["mixer"], ly.get("mlp"), f"l{i}.", layers[i]
            H, d, v, r = int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"])
            L.kind = 0 if ly["type"] == "latent_attention" else 1
            L.heads, L.dim, L.vdim, L.kv_rank, L.scale = H, d, v, r, float(m["scale"])
            L.q_rank = int(m["q_rank"]) if L.kind == 0 else 0
            src = m.get("kv_from")
            if src is None:
                self.arena_of[i] = len(ranks)
                ranks.append(r)
            else:
                self.arena_of[i] = self.arena_of[src]
            L.arena, L.writes_arena = self.arena_of[i], int(src is None)
            own = [sd[p + "mix.dkv"]] if src is None else []
            if L.kind == 0:
                w_in = torch.cat([sd[p + "mix.dq"]] + own, 0)
                L.q_norm, L.w_uq = self._p(sd[p + "mix.dq.norm"]), self._p(sd[p + "mix.uq"])
            else:
                w_in = torch.cat([sd[p + "mix.q"], sd[p + "mix.g"]] + own, 0)
            L.w_in = self._p(w_in)
            if src is None:
                L.kv_norm = self._p(sd[p + "mix.dkv.norm"])
            L.w_ukT = self._p(sd[p + "mix.uk"].reshape(H, d, r).transpose(1, 2))
            L.w_uv, L.w_o = self._p(sd[p + "mix.uv"]), self._p(sd[p + "mix.o"])
            for n in ("norm1", "norm1b"):
                setattr(L, n + "_w", self._p(sd[p + n]))
                setattr(L, n + "_b", self._p(sd[p + n + ".b"]))
            L.taps_w, L.rg1_w, L.rg1_b = self._p(sd[p + "canon1"]), self._p(sd[p + "rg1"]), self._p(sd[p + "rg1.b"])
            L.ff = 0
            if mlp is not None:
                L.ff = int(mlp["ff"])
                for n in ("norm2", "norm2b"):
                    setattr(L, n + "_w", self._p(sd[p + n]))
                    setattr(L, n + "_b", self._p(sd[p + n + ".b"]))
                L.w_ff_in = self._p(torch.cat([sd[p + "rg2"], sd[p + "mlp.up"]], 0))
                L.b_ff_in = self._p(torch.cat([sd[p + "rg2.b"], torch.zeros(L.ff, dtype=torch.bfloat16, device=dev)]))
                L.w_down, L.act = self._p(sd[p + "mlp.down"]), self._p(sd[p + "mlp.act"])
        self._layers, self.ranks = layers, ranks
        s = SeqModel()
        s.width, s.n_layers, s.taps, s.arith, s.eps = W, len(cfg.layers), cfg.taps, ARITH[arith], cfg.eps
        s.layers = C.cast(layers, C.POINTER(SeqLayer))
        s.final_w, s.final_b = self._p(sd["final.norm"]), self._p(sd["final.norm.b"])
        self.struct = s
        self.latent = [torch.zeros(self.n_seq, self.t_max, r, dtype=torch.float32, device=dev) for r in ranks]
        self.taps_state = torch.zeros(len(cfg.layers), self.n_seq, max(cfg.taps - 1, 1), W, dtype=torch.float32, device=dev)
        self._bind_state()
        self.block_rows = int(lib().mn_latent_attn_block_rows())
        self._ws, self._decode_tabs = {}, {}

    def _p(self, t):
        assert t.dtype == torch.bfloat16 and t.is_cuda
        t = t.contiguous()
        self._keep.append(t)
        return t.data_ptr()

    def _bind_state(self):
        self._latent_ptrs = _lib.ptr_array(self.latent)
        st = SeqState()
        st.latent, st.taps = C.cast(self._latent_ptrs, _lib.PP), self.taps_state.data_ptr()
        st.n_seq, st.t_max = self.n_seq, self.t_max
        self.state = st

    # ---- construction ---------------------------------------------------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, path, device="cuda", **kw):
        """A directory with config.json and *.safetensors (bf16 tensors under the checkpoint's names)."""
        from .infer import load_safetensors_dir
        cfg = PizitarConfig.from_pretrained(path)
        if not glob.glob(os.path.join(path, "*.safetensors")):
            raise FileNotFoundError(f"{path}: no *.safetensors")
        sd = {k: v.to(device, torch.bfloat16) for k, v in load_safetensors_dir(path).items() if v.is_floating_point()}
        return cls(cfg, sd, **kw)

    @classmethod
    def synthetic(cls, cfg, device="cuda", seed=0, **kw):
        """Random weights of the architecture (synth.py's rule by tensor name; activation coefficients near (0.6, 0.3, 0.2, 0))."""
        from .synth import synth_tensor
        sd = {}
        for k, shp in pizitar_param_shapes(cfg).items():
            if k.endswith(".b"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=0.02)
            elif k.endswith("mlp.act"):
                sd[k] = (torch.tensor([0.6, 0.3, 0.2, 0.0]) + synth_tensor(k, shp, seed, "cpu", torch.float32, 0.0, 0.05)).to(device, torch.bfloat16)
            elif k.endswith("canon1"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=0.3)
            elif k == "embed":
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=1.0)
            else:
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16)
        return cls(cfg, sd, **kw)

    # ---- cache sequences ----------------------------------------------------------------------------------------------------------
    def ensure_sequences(self, n_seq):
        """Grow the arenas and filter states to `n_seq` cache sequences; the existing ones keep their contents."""
        if n_seq <= self.n_seq:
            return
        per_seq = sum(self.t_max * r for r in self.ranks) * 4 + self.taps_state[:, 0].numel() * 4
        free, _ = torch.cuda.mem_get_info(self.device)
        if n_seq * per_seq > free:
            raise MemoryError(f"{n_seq} cache sequences at t_max = {self.t_max} need {n_seq * per_seq / 2**30:.1f} GiB, "
                              f"{free / 2**30:.1f} GiB free")
        for a, old in enumerate(self.latent):
            new = torch.zeros(n_seq, self.t_max, old.shape[2], dtype=torch.float32, device=self.device)
            new[:self.n_seq] = old
            self.latent[a] = new
        ts = torch.zeros((self.taps_state.shape[0], n_seq) + tuple(self.taps_state.shape[2:]), dtype=torch.float32, device=self.device)
        ts[:, :self.n_seq] = self.taps_state
        self.taps_state, self.n_seq = ts, n_seq
        self._bind_state()

    def release_sequences(self, n_keep):
        """Shrink back to the first `n_keep` cache sequences."""
        if n_keep >= self.n_seq:
            return
        self.latent = [a[:n_keep].clone() for a in self.latent]
        self.taps_state = self.taps_state[:, :n_keep].clone()
        self.n_seq = n_keep
        self._bind_state()

    def max_rows(self):
        return MAX_ROWS

    # ---- stepping -------------------------------------------------------------------------------------------------------------
    def _workspace(self, rows, max_len):
        key = torch.cuda.current_stream().cuda_stream
        need = int(lib().mn_seq_workspace_bytes(C.byref(self.struct), rows, max_len))
        if key not in self._ws or self._ws[key].numel() < need:
            self._ws[key] = torch.empty(need, dtype=torch.uint8, device=self.device)
        return self._ws[key]

    def step(self, x, row_seq, row_slot, row_back, row_len, blk_tab, max_len, out=None, trace=None, ws=None, distinct=False):
        """One pass of the stack over M rows.  x fp32 [M, width] (input embeddings); int32 device arrays per row (row r is
        position row_slot[r] of cache sequence row_seq[r], preceded in this pass by row_back[r] rows of its sequence, and attends
        row_len[r] = row_slot[r] + 1 slots); blk_tab int32 [n_blk, 2] cuts the rows into runs of <= block_rows consecutive rows of
        one sequence; max_len (host int) >= every row_len.  Appends the rows' latents and advances the filter states.
        trace: optional fp32 [layers, M, width] that receives the residual stream after every layer.
        distinct: every row is alone in its sequence (a decode step): the step fuses its gate / norm / filter launches.
        Returns the final norm's output [M, width] fp32."""
        M = x.shape[0]
        assert x.dtype == torch.float32 and x.is_cuda and x.stride(1) == 1 and x.shape[1] == self.cfg.width and 1 <= M <= MAX_ROWS
        for t in (row_seq, row_slot, row_back, row_len):
            assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous() and t.numel() >= M
        assert blk_tab.dtype == torch.int32 and blk_tab.is_cuda and blk_tab.is_contiguous() and blk_tab.shape[1] == 2
        assert 1 <= max_len <= self.t_max, f"{max_len} tokens exceed the arena (t_max = {self.t_max})"
        if out is None:
            out = torch.empty(M, self.cfg.width, dtype=torch.float32, device=self.device)
        if trace is not None:
            assert trace.dtype == torch.float32 and trace.is_contiguous() and tuple(trace.shape) == (len(self.cfg.layers), M, self.cfg.width)
        if ws is None:
            ws = self._workspace(M, max_len)
        check(lib().mn_seq_step(C.byref(self.struct), C.byref(self.state), ptr(x), x.stride(0), M, ptr(row_seq), ptr(row_slot),
                                ptr(row_back), ptr(row_len), ptr(blk_tab), blk_tab.shape[0], int(max_len), 1 if distinct else 0, ptr(out), ptr(trace),
                                ptr(ws), ws.numel(), current_stream()), "mn_seq_step")
        return out

    def forward_spans(self, x, spans, trace=False):
        """Rows of several sequences through the stack: spans = [(cache sequence, rows, tokens it already holds)] in row order,
        x fp32 [sum rows, width].  Runs in passes of <= max_rows() rows; a sequence cut by a pass boundary continues in the next
        pass.  Returns the final-norm hidden states [rows, width] (and the per-layer residual streams when trace)."""
        M = x.shape[0]
        assert sum(n for _, n, _ in spans) == M
        out = torch.empty(M, self.cfg.width, dtype=torch.float32, device=self.device)
        tr = torch.empty(len(self.cfg.layers), M, self.cfg.width, dtype=torch.float32, device=self.device) if trace else None
        starts = np.cumsum([0] + [n for _, n, _ in spans])
        for r0 in range(0, M, MAX_ROWS):
            r1 = min(M, r0 + MAX_ROWS)
            part = [(seq, min(starts[i + 1], r1) - max(starts[i], r0), past + max(starts[i], r0) - starts[i])
                    for i, (seq, n, past) in enumerate(spans) if min(starts[i + 1], r1) > max(starts[i], r0)]
            tabs = rows_of_spans([(int(s), int(n), int(p)) for s, n, p in part], self.block_rows)
            dev = {k: torch.from_numpy(v).to(self.device) for k, v in tabs.items() if k != "max_len"}
            ptr_tr = None
            if trace:
                ptr_tr = torch.empty(len(self.cfg.layers), r1 - r0, self.cfg.width, dtype=torch.float32, device=self.device)
            self.step(x[r0:r1], dev["row_seq"], dev["row_slot"], dev["row_back"], dev["row_len"], dev["blk_tab"], tabs["max_len"],
                      out=out[r0:r1], trace=ptr_tr, distinct=all(n == 1 for _, n, _ in part))
            if trace:
                tr[:, r0:r1] = ptr_tr
        return (out, tr) if trace else out

    def prefill(self, ids, seq=0, past=0):
        """Tokens ids (int tensor [T]) of ONE sequence from slot `past`; returns the hidden states [T, width]."""
        return self.forward_spans(self.embed(ids), [(seq, int(ids.numel()), past)])

    def decode_tables(self, B):
        """Static per-row tables of a lock-step decode step of B sequences (one row each): (row_back, blk_tab)."""
        if B not in self._decode_tabs:
            self._decode_tabs[B] = (torch.zeros(B, dtype=torch.int32, device=self.device),
                                    torch.stack([torch.arange(B, dtype=torch.int32), torch.ones(B, dtype=torch.int32)], 1).contiguous().to(self.device))
        return self._decode_tabs[B]

    def decode_graph(self, row_seq, row_slot, row_len):
        """A replayable lock-step decode step of B = len(row_seq) sequences (one row each): `DecodeGraph`."""
        return DecodeGraph(self, row_seq, row_slot, row_len)

    # ---- vocabulary -------------------------------------------------------------------------------------------------------------
    def embed(self, ids):
        return ops.bf16_to_f32(self.embed_w[ids.reshape(-1).to(self.device)])

    def logits(self, hidden):
        """Vocabulary projection + soft cap -> fp32 [M, vocab]."""
        hidden = hidden.contiguous()
        M, K = hidden.shape
        V = self.head_w.shape[0]
        out = torch.empty(M, V, dtype=torch.float32, device=self.device)
        ws = torch.empty(max(M * K * 2, 16), dtype=torch.uint8, device=self.device)
        check(lib().mn_seq_logits(ptr(hidden), K, M, ptr(self.head_w), V, K, float(self.cfg.logit_softcap or 0.0), ARITH[self.arith],
                                  ptr(out), V, ptr(ws), ws.numel(), current_stream()), "mn_seq_logits")
        return out

    def greedy(self, hidden):
        """Greedy pick of every row -> int64 [M] on the device.  The soft cap is increasing, so the arg-max of the uncapped
        product is the arg-max of the logits: the other decoder's fused vocabulary-projection + arg-max call serves here too
        (width a multiple of 8; otherwise through `logits`)."""
        if hidden.shape[1] % 8 == 0:
            return ops.lmhead_argmax(hidden.contiguous(), self.head_w)[0]
        return self.logits(hidden).argmax(-1)

    def sample(self, hidden, u, temperature=1.0, top_k=50, top_p=1.0):
        """Sampled pick of every row at the caller's uniforms u fp32 [M] (temperature -> top-k -> top-p -> one draw)."""
        return ops.sample_logits(self.logits(hidden), u, temperature, top_k, top_p)


class DecodeGraph:
    """One lock-step decode step (stack pass + advancing the rows' slots and lengths) captured as a HIP graph: a step of a small
    model is some twenty short launches per layer, and their host-side launch cost, not the kernels, bounds it.  The per-row
    state lives in device arrays that the graph's own last node advances, the input rows are copied into a fixed buffer, and the
    only host number baked in is an upper bound of the lengths (it sizes the attention's key splits), so one capture serves
    `span` tokens; `run` re-captures when the lengths pass the bound."""

    def __init__(self, dec, row_seq, row_slot, row_len, span=256):
        self.dec, self.span = dec, span
        self.row_seq, self.slot, self.len = row_seq, row_slot, row_len
        B = row_seq.numel()
        self.B = B
        self.back, self.blk = dec.decode_tables(B)
        self.x = torch.zeros(B, dec.cfg.width, dtype=torch.float32, device=dec.device)
        self.out = torch.empty(B, dec.cfg.width, dtype=torch.float32, device=dec.device)
        n = int(lib().mn_seq_workspace_bytes(C.byref(dec.struct), B, dec.t_max))
        self.ws = torch.empty(n, dtype=torch.uint8, device=dec.device)
        self.bound, self.graph = 0, None

    def _body(self):
        self.dec.step(self.x, self.row_seq, self.slot, self.back, self.len, self.blk, self.bound, out=self.out, ws=self.ws, distinct=True)
        check(lib().mn_rows_advance(ptr(self.slot), ptr(self.len), None, self.B, 1, current_stream()), "mn_rows_advance")

    def run(self, x, max_len):
        """x fp32 [B, width]: the new tokens' embeddings; max_len: host upper bound of the lengths after this step.
        Returns the hidden states [B, width] (a fixed buffer, overwritten by the next run)."""
        if self.graph is None or max_len > self.bound:
            self.bound = min(self.dec.t_max, (max_len + self.span - 1) // self.span * self.span)
            self.graph = torch.cuda.CUDAGraph()
            self.x.copy_(x)
            torch.cuda.synchronize(self.dec.device)
            snap = (self.slot.clone(), self.len.clone())
            with torch.cuda.graph(self.graph):
                self._body()
            # capture records, it does not run: the arrays are untouched, but restore them in case a runtime ever executes eagerly
            self.slot.copy_(snap[0])
            self.len.copy_(snap[1])
        self.x.copy_(x)
        self.graph.replay()
        return self.out


class PizitarForCausalLM:
    """Generation entry point: requests in, token ids out, in lock-step batches (the batching of the other decoder's
    `generate_text_batch`): all prompts share the prefill passes, then one pass per new token serves every live sequence."""

    def __init__(self, decoder: PizitarDecoder, eos_token_id=None):
        self.dec = decoder
        self.eos_token_id = eos_token_id
        self.slots = SequenceSlots(decoder)

    @classmethod
    def from_pretrained(cls, path, device="cuda", t_max=2048, arith="bf16", eos_token_id=None):
        return cls(PizitarDecoder.from_pretrained(path, device=device, t_max=t_max, arith=arith), eos_token_id)

    @torch.no_grad()
    def generate(self, prompts, max_new_tokens=16, do_sample=False, temperature=1.0, top_k=50, top_p=1.0, generator=None, sync_every=8,
                 use_graph=None):
        """prompts: list of token-id lists (unequal lengths allowed).  Greedy, or sampled (new token i of request b uses uniform
        [i, b] of one torch.rand(max_new_tokens, B) draw).  use_graph: run the decode steps as replays of a captured HIP graph
        (default: from 8 new tokens on).  Returns the new tokens of every request (cut after the first EOS)."""
        dec, dev = self.dec, self.dec.device
        B = len(prompts)
        lens = [len(p) for p in prompts]
        if min(lens) < 1 or max(lens) + max_new_tokens > dec.t_max:
            raise ValueError(f"prompts of 1 .. {dec.t_max - max_new_tokens} tokens (t_max = {dec.t_max})")
        seqs = [self.slots.alloc() for _ in range(B)]
        try:
            ids = torch.tensor([t for p in prompts for t in p], dtype=torch.long, device=dev)
            hid = dec.forward_spans(dec.embed(ids), [(s, n, 0) for s, n in zip(seqs, lens)])
            last = torch.tensor(np.cumsum(lens) - 1, dtype=torch.long, device=dev)
            hidden = hid[last].contiguous()
            row_seq = torch.tensor(seqs, dtype=torch.int32, device=dev)
            slot = torch.tensor(lens, dtype=torch.int32, device=dev)
            ln = slot + 1
            back, blk = dec.decode_tables(B)
            graph = dec.decode_graph(row_seq, slot, ln) if (max_new_tokens >= 8 if use_graph is None else use_graph) else None
            finished = torch.zeros(B, dtype=torch.bool, device=dev)
            uniforms = torch.rand(max_new_tokens, B, device=dev, generator=generator) if do_sample else None
            toks = []
            for i in range(max_new_tokens):
                tok = dec.sample(hidden, uniforms[i], temperature, top_k, top_p) if do_sample else dec.greedy(hidden)
                toks.append(tok)
                if self.eos_token_id is not None:
                    finished |= tok == self.eos_token_id
                    if (i + 1) % sync_every == 0 and bool(finished.all()):
                        break
                if i + 1 == max_new_tokens:
                    break
                if graph is not None:
                    hidden = graph.run(dec.embed(tok), max(lens) + i + 1)
                else:
                    hidden = dec.step(dec.embed(tok), row_seq, slot, back, ln, blk, max(lens) + i + 1, distinct=True)
                    check(lib().mn_rows_advance(ptr(slot), ptr(ln), None, B, 1, current_stream()), "mn_rows_advance")
            out = torch.stack(toks, 1).tolist()
        finally:
            for s in seqs:
                self.slots.release(s)
        res = []
        for row in out:
            if self.eos_token_id is not None and self.eos_token_id in row:
                row = row[:row.index(self.eos_token_id) + 1]
            res.append(row)
        return res
