"""Sakinex: a decoder-only language model of parallel-mixer layers, served by libmingnative's parallel-mixer step function
(mingnative.h section 10: mn_pmix_step).

Per layer run, with x the fp32 residual stream of a token, m = residual_mult and F_c the causal per-channel filter over the last
`canon.taps` inputs of the sequence:
    n  = RMS(x) w1,  h = n + F_1(n)
    left : q, k, v = W h, each channel through a short causal filter; rotary positions (YaRN frequencies) on the first rot.dims values
           of every q / k head, then every head divided by its root mean square; softmax over the tokens of a sliding window and over
           one mean key / value per whole block of `pool` tokens before the window; W_o on the heads
    right: minGRU  S = (1 - z) S + z c,  z = sigmoid(W_z h + b_z),  c = u + 1/2 (u >= 0) | sigmoid(u),  u = W_x h + b_x;  W_o (S silu(W_g h))
    x += m (left_scale left + right_scale right)
    n2 = RMS(x) w2,  h2 = n2 + F_2(n2)
    x += m (sum over the top experts of softmax(chosen router logits) expert(h2) + sigmoid(w_sg . h2) shared(h2)),  expert = W_d (silu(W_g .) * W_u .)
A range of layers may run several times with the same weights (`loop`): every run has its own caches and states, and the token's
embedding is added to x before each repeated pass.  Then RMS, and the vocabulary projection.

This module owns HBM residency, like bailing_moe.py and pizitar.py for the other decoders:
  * weights bf16; the projections that read the same rows are stacked at load ([q ; k ; v ; z ; x ; g], [shared gate ; shared up ;
    router ; shared gate logit]), the two output projections are joined along their inputs so that the scaled sum of both mixers is
    ONE product, and the experts lie in [experts, 2 ff, width] / [experts, width, ff] blocks;
  * per layer RUN: fp32 key / value arenas [n_seq, t_max, .], arenas of the pooled block means [n_seq, t_max / pool + 1, .], the
    filter states of both sublayers, the q / k / v filter state and the recurrent state [n_seq, .]; cache sequences are numbered
    as in the other decoders (`sequences.SequenceSlots`); a number that is given back is reused as it is: a row at position 0
    reads no state;
  * per-row int32 bookkeeping on the device, so a lock-step decode loop never syncs with the host.
`arith`: "bf16" = matrix products of steps above 8 rows on the bf16 MFMA kernels (fp32 accumulate), everything else fp32;
"f32" = fp32 FMA everywhere.
"""
import ctypes as C
import glob
import os

import torch

from . import _lib
from ._lib import PmixLayer, PmixModel, PmixState, check, current_stream, lib, ptr
from .configuration import SakinexConfig, sakinex_param_shapes
from .seq_lm import ARITH, SeqCausalLM, SeqDecoder


def rotary_table(rot, device):
    """-> (fp32 device tensor [dims / 2] of the pair frequencies, factor of cos and sin) of a `rot` dict."""
    dims = int(rot["dims"])
    sc = rot.get("scaling") or {}
    freq, mag = (C.c_float * (dims // 2))(), C.c_float()
    check(lib().mn_rotary_frequencies_host(dims, float(rot["base"]), float(sc.get("factor", 0.0)), float(sc.get("original", 0.0)),
                                           float(sc.get("fast", 0.0)), float(sc.get("slow", 0.0)), freq, C.byref(mag)), "mn_rotary_frequencies_host")
    return torch.tensor(list(freq), dtype=torch.float32, device=device), float(mag.value)


class SakinexDecoder(SeqDecoder):
    """Weights + per-run caches and states + the C-ABI tables of the stack."""

    def __init__(self, cfg: SakinexConfig, sd, t_max=2048, n_seq=1, arith="bf16"):
        """sd: {checkpoint tensor name: bf16 CUDA tensor}."""
        assert arith in ARITH, f"arith={arith!r}: 'bf16' or 'f32'"
        self.cfg, self.arith = cfg, arith
        missing = [k for k, shp in sakinex_param_shapes(cfg).items() if k not in sd or tuple(sd[k].shape) != tuple(shp)]
        if missing:
            raise ValueError(f"checkpoint does not fit the configuration: missing or mis-shaped tensors {missing[:8]}")
        dev = sd["embed"].device
        self.device = dev
        self.embed_w, self.head_w = sd["embed"].contiguous(), sd["head"].contiguous()
        self.t_max, self.n_seq = int(t_max), int(n_seq)
        W, taps = cfg.width, cfg.taps
        self._keep = []                                  # packed tensors the C tables point to
        bf = dict(dtype=torch.bfloat16, device=dev)
        layers = (PmixLayer * len(cfg.layers))()
        self.dims = []                                   # per layer: (key channels, value channels, q + k + v channels, conv, gru, pool)
        for i, ly in enumerate(cfg.layers):
            m, mlp, p, L = ly["mixer"], ly.get("mlp"), f"l{i}.", layers[i]
            lf, wr = m["left"], int(m["right"]["width"])
            H, G, d, e = int(lf["heads"]), int(lf["kv_heads"]), int(lf["dim"]), int(lf["vdim"])
            cqkv = (H + G) * d + G * e
            L.heads, L.kv_heads, L.dim, L.vdim, L.gru = H, G, d, e, wr
            L.conv = int(lf.get("conv") or 0)
            L.unit_qk, L.scale = 1, float(lf["scale"])
            L.left_scale, L.right_scale = float(m["left_scale"]), float(m["right_scale"])
            rot, mask = lf.get("rot"), lf.get("mask")
            L.rot_dims, L.rot_mag = 0, 1.0
            if rot:
                freq, mag = rotary_table(rot, dev)
                self._keep.append(freq)
                L.rot_dims, L.rot_mag, L.rot_freq = int(rot["dims"]), mag, freq.data_ptr()
            L.window = int(mask["size"]) if mask else 0
            L.pool = int(mask.get("pool") or 0) if mask else 0
            L.norm1 = self._p(sd[p + "norm1"])
            if taps:
                L.canon1 = self._p(sd[p + "canon1"])
            lp, rp = p + "mix.left.", p + "mix.right."
            L.w_in = self._p(torch.cat([sd[lp + "q"], sd[lp + "k"], sd[lp + "v"], sd[rp + "z"], sd[rp + "x"], sd[rp + "g"]], 0))
            L.b_in = self._p(torch.cat([torch.zeros(cqkv, **bf), sd[rp + "z.b"], sd[rp + "x.b"], torch.zeros(wr, **bf)]))
            if L.conv:
                L.w_conv = self._p(torch.cat([sd[lp + "q.conv"], sd[lp + "k.conv"], sd[lp + "v.conv"]], 0))
            L.w_out = self._p(torch.cat([sd[lp + "o"], sd[rp + "o"]], 1))
            L.experts = 0
            if mlp is not None:
                q = p + "mlp."
                E, top, ff = int(mlp["router"]["experts"]), int(mlp["router"]["top"]), int(mlp["expert"]["ff"])
                fs = int(mlp["shared"]["ff"]) if mlp.get("shared") else 0
                L.experts, L.top, L.ff, L.shared_ff = E, top, ff, fs
                L.norm2 = self._p(sd[p + "norm2"])
                if taps:
                    L.canon2 = self._p(sd[p + "canon2"])
                shared = [sd[q + "shared.gate"], sd[q + "shared.up"]] if fs else []
                pad = -(2 * fs + E + (1 if fs else 0)) % 8           # zero rows: the stack's row count a multiple of 8 (the wide GEMM's shapes)
                L.w_ff_in = self._p(torch.cat(shared + [sd[q + "router"]] + ([sd[q + "shared.sg"]] if fs else []) + [torch.zeros(pad, W, **bf)], 0))
                L.b_ff_in = self._p(torch.cat([torch.zeros(2 * fs, **bf), sd[q + "router.b"], torch.zeros((1 if fs else 0) + pad, **bf)]))
                if fs:
                    L.w_shared_down = self._p(sd[q + "shared.down"])
                L.w_gate_up = self._p(torch.stack([torch.cat([sd[f"{q}e{j}.gate"], sd[f"{q}e{j}.up"]], 0) for j in range(E)]))
                L.w_down = self._p(torch.stack([sd[f"{q}e{j}.down"] for j in range(E)]))
            self.dims.append((G * d, G * e, cqkv, L.conv, wr, L.pool))
        self._layers = layers
        runs = cfg.runs()
        self.runs = runs
        self.n_trace = len(runs)
        self._run_layer = (C.c_int32 * len(runs))(*[i for i, _ in runs])
        self._run_readd = (C.c_uint8 * len(runs))(*[int(a) for _, a in runs])
        s = PmixModel()
        s.width, s.n_layers, s.n_runs, s.taps, s.arith = W, len(cfg.layers), len(runs), taps, ARITH[arith]
        s.eps, s.mult = cfg.eps, cfg.residual_mult
        s.layers = C.cast(layers, C.POINTER(PmixLayer))
        s.run_layer, s.run_readd = self._run_layer, self._run_readd
        s.final_w = self._p(sd["final.norm"])
        self.struct = s
        pools = [d[5] for d in self.dims if d[5]]
        self.n_pool_max = self.t_max // min(pools) + 1 if pools else 1
        self.state_t = self._alloc_state(self.n_seq)
        self._bind_state()
        self.block_rows = int(lib().mn_window_attn_block_rows())
        self._ws, self._decode_tabs = {}, {}

    def _p(self, t):
        assert t.dtype == torch.bfloat16 and t.is_cuda
        t = t.contiguous()
        self._keep.append(t)
        return t.data_ptr()

    # ---- caches and states ---------------------------------------------------------------------------------------------------
    STATE_KEYS = ("k", "v", "pk", "pv", "canon", "conv", "gru")
    SEQ_AXIS = {"k": 0, "v": 0, "pk": 0, "pv": 0, "canon": 1, "conv": 0, "gru": 0}

    def _state_shapes(self, n_seq):
        """Per run: {name: shape or None}."""
        W, taps = self.cfg.width, self.cfg.taps
        out = []
        for li, _ in self.runs:
            ck, cv, cqkv, conv, wr, pool = self.dims[li]
            out.append({"k": (n_seq, self.t_max, ck), "v": (n_seq, self.t_max, cv),
                        "pk": (n_seq, self.n_pool_max, ck) if pool else None, "pv": (n_seq, self.n_pool_max, cv) if pool else None,
                        "canon": (2, n_seq, taps - 1, W) if taps > 1 else None,
                        "conv": (n_seq, conv - 1, cqkv) if conv > 1 else None, "gru": (n_seq, wr)})
        return out

    def _alloc_state(self, n_seq):
        return [{k: (None if shp is None else torch.zeros(shp, dtype=torch.float32, device=self.device)) for k, shp in run.items()}
                for run in self._state_shapes(n_seq)]

    def state_bytes_per_sequence(self):
        n = 0
        for run in self._state_shapes(1):
            for shp in run.values():
                if shp is not None:
                    n += 4 * int(torch.Size(shp).numel())
        return n

    def _bind_state(self):
        self._tabs = {k: _lib.ptr_array([run[k] for run in self.state_t]) for k in self.STATE_KEYS}
        st = PmixState()
        for k in self.STATE_KEYS:
            setattr(st, k, C.cast(self._tabs[k], _lib.PP))
        st.n_seq, st.t_max, st.n_pool_max = self.n_seq, self.t_max, self.n_pool_max
        self.state = st

    def ensure_sequences(self, n_seq):
        """Grow the caches and states to `n_seq` cache sequences; the existing ones keep their contents."""
        if n_seq <= self.n_seq:
            return
        need = n_seq * self.state_bytes_per_sequence()
        free, _ = torch.cuda.mem_get_info(self.device)
        if need > free:
            raise MemoryError(f"{n_seq} cache sequences at t_max = {self.t_max} need {need / 2**30:.1f} GiB, {free / 2**30:.1f} GiB free")
        new = self._alloc_state(n_seq)
        for old_run, new_run in zip(self.state_t, new):
            for k, t in old_run.items():
                if t is not None:
                    new_run[k].narrow(self.SEQ_AXIS[k], 0, self.n_seq).copy_(t)
        self.state_t, self.n_seq = new, n_seq
        self._bind_state()

    def release_sequences(self, n_keep):
        """Shrink back to the first `n_keep` cache sequences."""
        if n_keep >= self.n_seq:
            return
        self.state_t = [{k: (None if t is None else t.narrow(self.SEQ_AXIS[k], 0, n_keep).clone()) for k, t in run.items()}
                        for run in self.state_t]
        self.n_seq = n_keep
        self._bind_state()

    # ---- construction ---------------------------------------------------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, path, device="cuda", **kw):
        """A directory with config.json and *.safetensors (bf16 tensors under the checkpoint's names)."""
        from .infer import load_safetensors_dir
        cfg = SakinexConfig.from_pretrained(path)
        if not glob.glob(os.path.join(path, "*.safetensors")):
            raise FileNotFoundError(f"{path}: no *.safetensors")
        sd = {k: v.to(device, torch.bfloat16) for k, v in load_safetensors_dir(path).items() if v.is_floating_point()}
        return cls(cfg, sd, **kw)

    @classmethod
    def synthetic(cls, cfg, device="cuda", seed=0, **kw):
        """Random weights of the architecture (synth.py's rule by tensor name; filters of deviation 0.3, biases 0.02)."""
        from .synth import synth_tensor
        sd = {}
        for k, shp in sakinex_param_shapes(cfg).items():
            if k.endswith(".b"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=0.02)
            elif k.endswith(".conv") or k.endswith("canon1") or k.endswith("canon2"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=0.3)
            elif k == "embed":
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=1.0)
            elif "norm" in k:
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=1.0, std=0.05)
            else:
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=shp[-1] ** -0.5)
        return cls(cfg, sd, **kw)

    # ---- stepping -------------------------------------------------------------------------------------------------------------
    def _workspace_bytes(self, rows, max_len):
        return lib().mn_pmix_workspace_bytes(C.byref(self.struct), rows)

    def max_rows(self):
        """Rows of one pass: the (row, expert) pairs of a pass are at most 65535."""
        top = max([int(ly["mlp"]["router"]["top"]) for ly in self.cfg.layers if ly.get("mlp")] or [1])
        return max(1, min(super().max_rows(), 65535 // top))

    def step(self, x, row_seq, row_slot, row_back, row_len=None, blk_tab=None, max_len=None, out=None, trace=None, ws=None, distinct=False):
        """One pass of the stack over M rows.  x fp32 [M, width] (input embeddings); int32 device arrays per row (row r is position
        row_slot[r] of cache sequence row_seq[r], preceded in this pass by row_back[r] rows of its sequence); blk_tab int32 [n_blk, 2]
        cuts the rows into runs of <= block_rows consecutive rows of one sequence (not read when distinct); row_len is the other
        decoder's table and is not read here; max_len (host int) >= every position + 1 (default: the cache's length).  Appends the rows' keys
        and values, completes pooled blocks, advances the filter and recurrent states.  trace: optional fp32 [runs, M, width] that
        receives the residual stream after every layer run.  distinct: every row is alone in its sequence (a decode step): the step
        fuses its residual add / norm / filter launches.  Returns the final norm's output [M, width] fp32."""
        M = x.shape[0]
        assert x.dtype == torch.float32 and x.is_cuda and x.stride(1) == 1 and x.shape[1] == self.cfg.width and 1 <= M <= self.max_rows()
        for t in (row_seq, row_slot, row_back):
            assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous() and t.numel() >= M
        max_len = self.t_max if max_len is None else int(max_len)
        assert 1 <= max_len <= self.t_max, f"{max_len} tokens exceed the cache (t_max = {self.t_max})"
        if not distinct:
            assert blk_tab is not None and blk_tab.dtype == torch.int32 and blk_tab.is_cuda and blk_tab.is_contiguous() and blk_tab.shape[1] == 2
        if out is None:
            out = torch.empty(M, self.cfg.width, dtype=torch.float32, device=self.device)
        if trace is not None:
            assert trace.dtype == torch.float32 and trace.is_contiguous() and tuple(trace.shape) == (self.n_trace, M, self.cfg.width)
        if ws is None:
            ws = self._workspace(M, max_len)
        check(lib().mn_pmix_step(C.byref(self.struct), C.byref(self.state), ptr(x), x.stride(0), M, ptr(row_seq), ptr(row_slot), ptr(row_back),
                                 None if distinct else ptr(blk_tab), M if distinct else blk_tab.shape[0], max_len, 1 if distinct else 0, ptr(out),
                                 ptr(trace), ptr(ws), ws.numel(), current_stream()), "mn_pmix_step")
        return out


class SakinexForCausalLM(SeqCausalLM):
    """`SeqCausalLM` over a `SakinexDecoder`."""

    @classmethod
    def from_pretrained(cls, path, device="cuda", t_max=2048, arith="bf16", eos_token_id=None):
        return cls(SakinexDecoder.from_pretrained(path, device=device, t_max=t_max, arith=arith), eos_token_id)
