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
from .seq_lm import ARITH, MAX_ROWS, DecodeGraph, SeqCausalLM, SeqDecoder  # noqa: F401


class PizitarDecoder(SeqDecoder):
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
        self.n_trace = len(cfg.layers)

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

    # ---- stepping -------------------------------------------------------------------------------------------------------------
    def max_rows(self):
        return MAX_ROWS

    def _workspace_bytes(self, rows, max_len):
        return lib().mn_seq_workspace_bytes(C.byref(self.struct), rows, max_len)

    def step(self, x, row_seq, row_slot, row_back, row_len, blk_tab, max_len, out=None, trace=None, ws=None, distinct=False):
        """One pass of the stack over M rows.  x fp32 [M, width] (input embeddings); int32 device arrays per row (row r is
        position row_slot[r] of cache sequence row_seq[r], preceded in this pass by row_back[r] rows of its sequence, and attends
        row_len[r] = row_slot[r] + 1 slots); blk_tab int32 [n_blk, 2] cuts the rows into runs of <= block_rows consecutive rows of
        one sequence; max_len (host int) >= every row_len.  Appends the rows' latents and advances the filter states.
        trace: optional fp32 [layers, M, width] that receives the residual stream after every layer.
        distinct: every row is alone in its sequence (a decode step): the step fuses its gate / norm / filter launches.
        Returns the final norm's output [M, width] fp32."""
        M = x.shape[0]
        assert x.dtype == torch.float32 and x.is_cuda and x.stride(1) == 1 and x.shape[1] == self.cfg.width and 1 <= M <= self.max_rows()
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


class PizitarForCausalLM(SeqCausalLM):
    """`SeqCausalLM` over a `PizitarDecoder`."""

    @classmethod
    def from_pretrained(cls, path, device="cuda", t_max=2048, arith="bf16", eos_token_id=None):
        return cls(PizitarDecoder.from_pretrained(path, device=device, t_max=t_max, arith=arith), eos_token_id)
