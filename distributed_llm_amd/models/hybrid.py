"""Layer-list decoder (Filevik): every layer has a token mixer (Mamba-1 selective scan, retention,
latent attention) and an optional mixture-of-experts feed-forward, in the order config.json gives.

The residual stream lives in f32; each sublayer reads its rounding to the model dtype and adds
``rmsnorm(sublayer(x)) * w`` (ops.seqmix.norm_resadd: the f32 add, the norm and the rounded copy in
one launch).  Projections run on the framework's GEMMs (ops.linear; the vendor GEMM for shapes
they do not take and for f32 models), everything between them on the HIP kernels of ops.seqmix:

  mamba1     in-proj -> causal conv + SiLU (reads the slot's last inputs) -> x-proj -> dt-proj ->
             selective scan (f32 state per slot, softplus / decay / gate in f32; refills the
             convolution state) -> out-proj
  retention  one fused q|k|v|gate projection -> decayed linear attention (rotate-half positions,
             f32 state per slot, unit-RMS heads, SiLU gate in the kernel) -> out-proj
  latent     one fused down projection (query latent | key/value latent | shared rotated key) ->
             query up-projection -> the key up-projection is absorbed into the query (per-head
             batched GEMM), so attention runs over the cached latent alone (paged, written by a
             kernel that norms the latent and rotates the shared key) -> value up-projection per
             head -> out-proj
  experts    fused router (f32 softmax top-k, renormalised) -> grouped squared-ReLU expert GEMMs, or
             the dense form (all experts' columns, unused ones gated to zero) for f32 models and
             unaligned widths -> plus the shared expert

Per-sequence state lives in slots owned by the engine (its batch rows); paged latents use the
engine's block tables.  No tensor parallelism.
"""
from __future__ import annotations

import math
import os
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import seqmix
from ..parallel.comm import SINGLE, ParallelContext
from .configs import HybridConfig, LayerSpec, MixerSpec, MoESpec


def _mm(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x @ w.T: the framework's tuned GEMM where it takes the shape, else the vendor GEMM."""
    if (x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1
            and x.shape[1] % 64 == 0 and w.shape[0] % 64 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.is_contiguous()):
        return ops.linear(x, w)
    return F.linear(x, w)


class HybridModel:
    fused = False                      # no folded-norm GEMM epilogues (engine autotune hook)
    has_recurrent_state = True
    attn_geometry = None               # no softmax-attention split-K workspace

    def __init__(self, cfg: HybridConfig, device="cuda", dtype=torch.bfloat16, par: ParallelContext = SINGLE,
                 seed: int = 0, weights: Optional[str] = None, init_std: float = 0.02):
        if par.tp_size > 1:
            raise ValueError(f"{cfg.name}: layer-list models run on one GPU (no tensor parallelism)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("dtype must be bfloat16 or float32")
        self.cfg, self.device, self.dtype, self.par = cfg, torch.device(device), dtype, par
        self.has_recurrent_state = any(L.mixer.recurrent for L in cfg.layers)
        self.layers: List[Dict[str, torch.Tensor]] = []
        self.tap: Optional[list] = None      # debugging: residual stream after every layer
        self._rot: Dict[Tuple[int, float], torch.Tensor] = {}
        self._max_pos = 0
        raw = self._load(weights) if weights else self._random(seed, init_std)
        self._place(raw)
        self.ensure_positions(2048)

    # ------------------------------------------------------------------ weights
    def _random(self, seed: int, std: float) -> Dict[str, torch.Tensor]:
        """Seeded random tensors under the checkpoint's names (benchmarks, tests)."""
        g = torch.Generator().manual_seed(seed)
        cfg, W = self.cfg, self.cfg.hidden
        t: Dict[str, torch.Tensor] = {}

        def rnd(*shape, s=std):
            return torch.randn(*shape, generator=g) * s

        def lin(n_out, n_in):
            return rnd(n_out, n_in, s=1.0 / math.sqrt(n_in))

        t["embed"] = rnd(cfg.vocab, W, s=1.0)
        t["head"] = lin(cfg.vocab, W)
        t["final.norm"] = torch.ones(W)
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L.mixer
            t[p + "norm1"] = torch.ones(W)
            if m.kind == "mamba1":
                t[p + "mix.in"] = lin(2 * m.inner, W)
                t[p + "mix.conv"] = rnd(m.inner, m.conv, s=1.0 / math.sqrt(m.conv))
                t[p + "mix.conv.b"] = rnd(m.inner, s=0.1)
                t[p + "mix.x"] = lin(m.dt_rank + 2 * m.state, m.inner)
                t[p + "mix.dt"] = lin(m.inner, m.dt_rank)
                dt = torch.exp(torch.rand(m.inner, generator=g) * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
                t[p + "mix.dt.b"] = dt + torch.log(-torch.expm1(-dt))
                t[p + "mix.A_log"] = torch.log(torch.arange(1, m.state + 1, dtype=torch.float32))[None, :].repeat(m.inner, 1)
                t[p + "mix.D"] = torch.ones(m.inner)
                t[p + "mix.o"] = lin(W, m.inner)
            elif m.kind == "retention":
                t[p + "mix.q"], t[p + "mix.k"] = lin(m.heads * m.dim, W), lin(m.heads * m.dim, W)
                t[p + "mix.v"], t[p + "mix.g"] = lin(m.heads * m.vdim, W), lin(m.heads * m.vdim, W)
                t[p + "mix.o"] = lin(W, m.heads * m.vdim)
            else:
                t[p + "mix.dq"], t[p + "mix.dq.norm"] = lin(m.q_rank, W), torch.ones(m.q_rank)
                t[p + "mix.uq"] = lin(m.heads * (m.dim + m.rot_dim), m.q_rank)
                t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = lin(m.kv_rank + m.rot_dim, W), torch.ones(m.kv_rank)
                t[p + "mix.uk"], t[p + "mix.uv"] = lin(m.heads * m.dim, m.kv_rank), lin(m.heads * m.vdim, m.kv_rank)
                t[p + "mix.o"] = lin(W, m.heads * m.vdim)
            f = L.mlp
            if f is not None:
                t[p + "norm2"] = torch.ones(W)
                t[p + "mlp.router"] = lin(f.experts, W)
                for e in range(f.experts):
                    t[p + f"mlp.e{e}.up"], t[p + f"mlp.e{e}.down"] = lin(f.ff, W), lin(W, f.ff)
                if f.shared_ff:
                    t[p + "mlp.shared.up"], t[p + "mlp.shared.down"] = lin(f.shared_ff, W), lin(W, f.shared_ff)
        return t

    @staticmethod
    def _load(path: str) -> Dict[str, torch.Tensor]:
        from safetensors import safe_open
        files = [path] if os.path.isfile(path) else sorted(
            os.path.join(path, f) for f in os.listdir(path) if f.endswith(".safetensors"))
        out: Dict[str, torch.Tensor] = {}
        for f in files:
            with safe_open(f, framework="pt", device="cpu") as fh:
                for k in fh.keys():
                    out[k] = fh.get_tensor(k)
        return out

    def _place(self, t: Dict[str, torch.Tensor]) -> None:
        """Checkpoint tensors -> device layouts (fused projections, per-head batched matrices,
        f32 copies of what the recurrences read)."""
        cfg, dev, dt = self.cfg, self.device, self.dtype
        put = lambda x: x.to(dev, dt).contiguous()
        f32 = lambda x: x.to(dev, torch.float32).contiguous()
        W = cfg.hidden
        self.embed, self.lm_head, self.final_norm = put(t["embed"]), put(t["head"]), f32(t["final.norm"])
        if tuple(self.embed.shape) != (cfg.vocab, W) or tuple(self.lm_head.shape) != (cfg.vocab, W):
            raise ValueError("embed / head do not fit config vocab x width")
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L.mixer
            D: Dict[str, torch.Tensor] = {"norm1": f32(t[p + "norm1"])}
            if m.kind == "mamba1":
                D["in"], D["x"], D["dt"], D["o"] = (put(t[p + "mix." + n]) for n in ("in", "x", "dt", "o"))
                D["conv"], D["conv_b"] = f32(t[p + "mix.conv"]), f32(t[p + "mix.conv.b"])
                D["dt_b"], D["D"] = f32(t[p + "mix.dt.b"]), f32(t[p + "mix.D"])
                D["A"] = -torch.exp(f32(t[p + "mix.A_log"]))
                assert tuple(D["A"].shape) == (m.inner, m.state) and tuple(D["conv"].shape) == (m.inner, m.conv)
            elif m.kind == "retention":
                D["qkvg"] = put(torch.cat([t[p + "mix." + n] for n in "qkvg"], 0))
                D["o"] = put(t[p + "mix.o"])
                D["decay"] = torch.tensor(m.decay, dtype=torch.float32, device=dev)
                assert D["decay"].numel() == m.heads
            else:
                D["dqkv"] = put(torch.cat([t[p + "mix.dq"], t[p + "mix.dkv"]], 0))
                D["dq_norm"], D["dkv_norm"] = f32(t[p + "mix.dq.norm"]), f32(t[p + "mix.dkv.norm"])
                D["uq"], D["o"] = put(t[p + "mix.uq"]), put(t[p + "mix.o"])
                D["uk"] = put(t[p + "mix.uk"].view(m.heads, m.dim, m.kv_rank))                       # [H, d, r]
                D["uvT"] = put(t[p + "mix.uv"].view(m.heads, m.vdim, m.kv_rank).transpose(1, 2))    # [H, r, dv]
            f = L.mlp
            if f is not None:
                D["norm2"] = f32(t[p + "norm2"])
                D["router"] = put(t[p + "mlp.router"])
                w1 = torch.stack([t[p + f"mlp.e{e}.up"] for e in range(f.experts)])       # [E, ff, W]
                w2 = torch.stack([t[p + f"mlp.e{e}.down"] for e in range(f.experts)])     # [E, W, ff]
                D["w1"] = put(w1)
                grouped = (dt == torch.bfloat16 and dev.type == "cuda" and W % 32 == 0 and f.ff % 32 == 0
                           and f.experts <= 64)
                if grouped or dev.type != "cuda":
                    D["w2"] = put(w2)
                else:   # dense form: one down projection over every expert's columns
                    D["w2d"] = put(w2.permute(1, 0, 2).reshape(W, f.experts * f.ff))
                if f.shared_ff:
                    D["sh_up"], D["sh_down"] = put(t[p + "mlp.shared.up"]), put(t[p + "mlp.shared.down"])
            self.layers.append(D)

    def weight_bytes(self) -> int:
        n = sum(x.numel() * x.element_size() for x in (self.embed, self.lm_head, self.final_norm))
        return n + sum(x.numel() * x.element_size() for L in self.layers for x in L.values())

    def decode_read_bytes(self, top_only: bool = True) -> int:
        """Weight bytes one decode token reads (routed experts: ``top`` of them)."""
        n = self.lm_head.numel() * self.lm_head.element_size()
        for L, S in zip(self.layers, self.cfg.layers):
            for k, x in L.items():
                b = x.numel() * x.element_size()
                if k in ("w1", "w2", "w2d") and top_only and S.mlp is not None:
                    b = b * S.mlp.top // S.mlp.experts
                n += b
        return n

    # ------------------------------------------------------------------ positions, caches
    def ensure_positions(self, n: int) -> None:
        """cos | sin tables (f64 on the host, stored f32) for positions < n of every rotation used."""
        if n <= self._max_pos:
            return
        self._max_pos = n
        for L in self.cfg.layers:
            r = L.mixer.rot
            if r is not None and r.dims > 0:
                self._rot[(r.dims, r.base)] = ops.rope_cos_sin(n, r.dims, r.base, self.device)

    def _table(self, m: MixerSpec) -> torch.Tensor:
        return self._rot[(m.rot.dims, m.rot.base)]

    def block_bytes(self, block_size: int) -> int:
        """Bytes of one paged block over all layers (latent attention layers only)."""
        it = torch.empty((), dtype=self.dtype).element_size()
        return sum(block_size * (L.mixer.kv_rank + L.mixer.rot_dim) * it for L in self.cfg.layers
                   if L.mixer.kind == "latent_attention")

    def alloc_caches(self, num_blocks: int, block_size: int, slots: int) -> List[tuple]:
        """Per layer: (paged latent [blocks, block, rank + rot],) or the recurrent state of ``slots``
        sequences: (conv inputs [slots, taps - 1, inner], scan state [slots, inner, state] f32) /
        (retention state [slots, heads, dim, vdim] f32,)."""
        dev, out = self.device, []
        for L in self.cfg.layers:
            m = L.mixer
            if m.kind == "mamba1":
                out.append((torch.zeros((slots, max(m.conv - 1, 0), m.inner), dtype=self.dtype, device=dev),
                            torch.zeros((slots, m.inner, m.state), dtype=torch.float32, device=dev)))
            elif m.kind == "retention":
                out.append((torch.zeros((slots, m.heads, m.dim, m.vdim), dtype=torch.float32, device=dev),))
            else:
                out.append((torch.zeros((num_blocks, block_size, m.kv_rank + m.rot_dim), dtype=self.dtype, device=dev),))
        return out

    # ------------------------------------------------------------------ mixers
    def _mamba(self, L, m: MixerSpec, x, meta, cache):
        conv_state, ssm_state = cache
        rows = meta.state_rows
        xz = _mm(x, L["in"])
        xc = seqmix.causal_conv_silu(xz, L["conv"], L["conv_b"], conv_state, meta.qstart, meta.qlen, meta.ctx, rows)
        dbc = _mm(xc, L["x"])
        dt_raw = _mm(dbc[:, :m.dt_rank], L["dt"])
        y = seqmix.selective_scan(xc, dt_raw, L["dt_b"], L["A"], dbc, m.dt_rank, L["D"], xz, ssm_state, conv_state,
                                  meta.qstart, meta.qlen, meta.ctx, rows)
        return _mm(y, L["o"])

    def _retention(self, L, m: MixerSpec, x, positions, meta, cache):
        qkvg = _mm(x, L["qkvg"])
        rot = m.rot.dims if m.rot is not None else 0
        table = self._table(m) if rot else self._any_table()
        o = seqmix.retention(qkvg, m.heads, m.dim, m.vdim, table, rot, L["decay"], cache[0], self.cfg.rms_eps,
                             positions, meta.qstart, meta.qlen, meta.ctx, meta.state_rows)
        return _mm(o, L["o"])

    def _any_table(self) -> torch.Tensor:
        if not self._rot:
            self._rot[(2, 1.0)] = ops.rope_cos_sin(self._max_pos, 2, 1.0, self.device)
        return next(iter(self._rot.values()))

    def _latent(self, L, m: MixerSpec, x, positions, meta, cache):
        T, H, eps = x.shape[0], m.heads, self.cfg.rms_eps
        down = _mm(x, L["dqkv"])
        cq = seqmix.rms_rows(down[:, :m.q_rank], L["dq_norm"], eps)
        q = _mm(cq, L["uq"])                                            # [T, H (dim + rot)]
        table = self._table(m)
        seqmix.latent_kv_write(down[:, m.q_rank:], m.kv_rank, L["dkv_norm"], eps, positions, table, meta.slots,
                               cache[0])
        qn = q.view(T, H, m.dim + m.rot_dim)[:, :, :m.dim].transpose(0, 1)
        qa = torch.bmm(qn, L["uk"])                                     # key up-projection absorbed: [H, T, rank]
        rows = (seqmix.LAT_ROWS if meta.host_qlen is None else
                seqmix.latent_rows(x, m.kv_rank, m.rot_dim, T, len(meta.host_qlen)))
        ts, tr = meta.latent_tiles(H, self.device, rows)
        lat = seqmix.latent_attention(qa, q, m.dim, m.rot_dim, positions, table, cache[0], meta.block_tables,
                                      meta.qstart, meta.qlen, meta.ctx, ts, tr, m.scale, rows=rows)
        o = torch.bmm(lat, L["uvT"])                                    # [H, T, vdim]
        return _mm(o.transpose(0, 1).reshape(T, H * m.vdim), L["o"])

    def _experts(self, L, f: MoESpec, x):
        if f.experts > 64 or f.top > 8:      # beyond the router kernels' register budget: library top-k
            val, ids = torch.topk(torch.softmax(F.linear(x.float(), L["router"].float()), -1), f.top, -1)
            ids, w = ids.to(torch.int32), val / (val.sum(-1, keepdim=True) + 1e-20)
        elif x.is_cuda and x.dtype == torch.bfloat16:
            ids, w = ops.moe_router(x, L["router"], f.top)      # f32 logits, softmax over the chosen = s / sum s
        else:
            ids, w = ops.moe_gate(F.linear(x.float(), L["router"].float()), f.top)
        w = w * f.scale
        if "w2" in L and (not x.is_cuda or seqmix.moe_ffn_relu2_ok(x, L["w1"])):
            y = seqmix.moe_ffn_relu2(x, ids, w, L["w1"], L["w2"])
        else:
            if "w2d" not in L:
                L["w2d"] = L["w2"].permute(1, 0, 2).reshape(x.shape[1], -1).contiguous()
            g = seqmix.dense_gate(ids, w, f.experts)
            a = seqmix.relu2_scale(_mm(x, L["w1"].view(f.experts * f.ff, -1)), g, f.ff)
            y = _mm(a, L["w2d"])
        if f.shared_ff:
            y = y + _mm(seqmix.relu2_scale(_mm(x, L["sh_up"])), L["sh_down"])
        return y

    # ------------------------------------------------------------------ forward
    def hidden_states(self, input_ids: torch.Tensor, positions: torch.Tensor, meta, kv_caches: List[tuple],
                      scatter: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> torch.Tensor:
        """Final-normed hidden states of the packed rows ``meta.last_idx`` (every row when
        ``meta.all_last``): [S, width] in the model dtype."""
        cfg, eps = self.cfg, self.cfg.rms_eps
        if scatter is not None:
            ops.scatter_pairs(*scatter)
        if self.dtype == torch.bfloat16:
            if cfg.hidden % 8 == 0:
                xl = ops.embedding(input_ids, self.embed)
            else:      # the gather kernel moves 16-byte vectors
                xl = self.embed.index_select(0, input_ids.long())
            x = xl.float()
        else:
            x = self.embed.index_select(0, input_ids.long())
            xl = None
        for L, S, cache in zip(self.layers, cfg.layers, kv_caches):
            m = S.mixer
            h = x if xl is None else xl
            if m.kind == "mamba1":
                y = self._mamba(L, m, h, meta, cache)
            elif m.kind == "retention":
                y = self._retention(L, m, h, positions, meta, cache)
            else:
                y = self._latent(L, m, h, positions, meta, cache)
            seqmix.norm_resadd(y, L["norm1"], eps, x, xl)
            if S.mlp is not None:
                y = self._experts(L, S.mlp, x if xl is None else xl)
                seqmix.norm_resadd(y, L["norm2"], eps, x, xl)
            if self.tap is not None:
                self.tap.append(x.clone())
        sel = x if meta.all_last else x.index_select(0, meta.last_idx)
        return seqmix.rms_rows(sel, self.final_norm, eps, out_dtype=self.dtype)

    def logits(self, hidden: torch.Tensor) -> torch.Tensor:
        lg = _mm(hidden, self.lm_head)
        return lg if self.cfg.logit_scale == 1.0 else lg * self.cfg.logit_scale

    def logits_f32(self, hidden: torch.Tensor) -> torch.Tensor:
        return _mm(hidden, self.lm_head).float() * self.cfg.logit_scale

    def _sampler_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """bf16 logits [S, vocab] whose rows start 16-byte aligned (the sampler kernels read vectors)."""
        lg = self.logits(hidden)
        V = lg.shape[1]
        if V % 8 == 0 or not lg.is_cuda:
            return lg.to(torch.bfloat16)
        buf = torch.zeros((lg.shape[0], (V + 7) // 8 * 8), dtype=torch.bfloat16, device=lg.device)
        buf[:, :V].copy_(lg)
        return buf[:, :V]

    def greedy(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.argmax(self._sampler_logits(hidden))

    def sample(self, hidden, temperature, top_p, top_k, seed, out):
        return ops.sample_rows(self._sampler_logits(hidden), temperature, top_p, top_k, seed, out=out)

    def topk_candidates(self, hidden: torch.Tensor, k: int):
        v, i = torch.topk(self.logits(hidden).float(), min(k, self.cfg.vocab), dim=-1)
        return v.contiguous(), i.contiguous()
