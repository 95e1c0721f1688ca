"""A Gemma-2B-shaped decoder-only transformer step (batch 1) on int4 group-32 weights, built from the library's
GEMV and the small decode kernels.  Every launch goes through the C ABI on torch's current stream; position
and token live in device memory, so the whole step can be captured once in a HIP graph and replayed.

Model conventions are this build's plain choices (the benchmark text fixes shapes only): RMSNorm y = x/rms*w,
rotate-half RoPE base 10000, multi-query attention with one KV head, GeGLU with tanh-GELU, tied int4
embedding / output table without embedding scaling or logit soft-capping.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from . import _lib
from .formats import QWeightInt4G32, quantize_int4_g32


@dataclass
class DecoderConfig:
    n_layers: int = 18
    d: int = 2048
    hq: int = 8
    dh: int = 256
    ffn: int = 16384
    vocab: int = 256000
    max_ctx: int = 4096
    eps: float = 1e-6
    rope_base: float = 10000.0


def random_weights(cfg: DecoderConfig, seed: int, device) -> Dict:
    """Random-init fp32 weights ~N(0, 0.02) quantised to int4 group-32 (absmax/7 per group); norms ~1."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)

    def q(n, k):
        # generate and quantise in slabs to bound memory (the output table is 2 GB in fp32)
        packed, scale = [], []
        for r0 in range(0, n, 32768):
            w = torch.randn(min(32768, n - r0), k, device=device, generator=g) * 0.02
            qw = quantize_int4_g32(w)
            packed.append(qw.packed)
            scale.append(qw.scale)
        return QWeightInt4G32(torch.cat(packed), torch.cat(scale))

    def norm():
        return (1.0 + 0.1 * torch.randn(cfg.d, device=device, generator=g)).float()

    layers = []
    for _ in range(cfg.n_layers):
        layers.append({
            "ln1": norm(), "wqkv": q((cfg.hq + 2) * cfg.dh, cfg.d), "wo": q(cfg.d, cfg.hq * cfg.dh),
            "ln2": norm(), "wgu": q(2 * cfg.ffn, cfg.d), "wd": q(cfg.d, cfg.ffn),
        })
    return {"layers": layers, "lnf": norm(), "emb": q(cfg.vocab, cfg.d)}


def save_weights(path: str, cfg: DecoderConfig, weights: Dict) -> None:
    """Writes a decoder's weights and configuration to one weight-container file (chadslab_amd.wfile)."""
    from dataclasses import asdict

    from . import wfile

    flat = {"lnf": weights["lnf"], "emb": weights["emb"]}
    for li, L in enumerate(weights["layers"]):
        for k, v in L.items():
            flat["layers.%d.%s" % (li, k)] = v
    wfile.save(path, flat, meta={"decoder_config": asdict(cfg)})


def load_weights(path: str, device):
    """Inverse of save_weights: returns (DecoderConfig, weights) with every tensor on `device`."""
    from . import wfile

    cfg = DecoderConfig(**wfile.read_header(path)["meta"]["decoder_config"])
    flat = wfile.load(path, device)
    layers = [{k: flat["layers.%d.%s" % (li, k)] for k in ("ln1", "wqkv", "wo", "ln2", "wgu", "wd")} for li in range(cfg.n_layers)]
    return cfg, {"layers": layers, "lnf": flat["lnf"], "emb": flat["emb"]}


class QuantDecoder:
    def __init__(self, cfg: DecoderConfig, weights: Dict, device="cuda:0", release_gate_up: bool = False):
        """release_gate_up: once the row-interleaved copy of a layer's gate/up matrix exists (GeGLU folded into that
        projection), delete the matrix from the `weights` dict that was handed in: the step never reads it again, and
        at the benchmark's shape the copies are 0.68 GB beside 1.45 GB of weights.  The dict can then no longer be
        saved or given to another decoder."""
        if not torch.cuda.is_available():
            raise RuntimeError("QuantDecoder needs the GPU (there is no CPU path)")
        self.cfg, self.w, self.dev = cfg, weights, torch.device(device)
        self.lib = _lib.load()
        f32, bf16, i32 = torch.float32, torch.bfloat16, torch.int32
        z = lambda n, dt: torch.zeros(n, dtype=dt, device=self.dev)  # noqa: E731
        c = cfg
        self.x, self.x2, self.xn = z(c.d, f32), z(c.d, f32), z(c.d, bf16)  # the residual stream ping-pongs between x and x2
        self.fused_norm1 = c.d % 256 == 0 and c.d <= 2048  # first norm of a layer folded into the qkv projection
        self.qkv, self.q = z((c.hq + 2) * c.dh, f32), z(c.hq * c.dh, f32)
        # the combination of the attention partials folded into the o projection, which then leaves one partial vector
        # per pair of heads for the next residual add (the entry point's rules: dh = 256, an even hq; the adds that
        # follow take up to four vectors; the entry point clears the vectors itself before its heads add into them)
        self.fused_oproj = c.dh == 256 and c.hq in (2, 4, 6, 8) and c.max_ctx <= 65536
        self.att, self.ao = z(c.hq * c.dh, bf16), z((c.hq // 2 if self.fused_oproj else 1) * c.d, f32)
        # the down projection has few rows and a long K: split it over K when that fills the chip better
        self.ksplit = next((s for s in (4, 2) if c.ffn % (s * 4096) == 0), 1)
        self.gu, self.h, self.dn = z(2 * c.ffn, f32), z(c.ffn, bf16), z(self.ksplit * c.d, f32)
        self.logits = z(c.vocab, f32)
        # GeGLU folded into the gate+up projection: the kernel wants the gate and the up row of a feature next to each
        # other, so the decoder keeps a row-interleaved copy of each layer's [2F, d] matrix (made here, once; the
        # matrices handed in keep the gate-rows-then-up-rows order of the file format)
        # (the entry point's own rules: an even number of rows, K a multiple of 256 up to 2048, N * K / 2 below 2^31)
        self.fused_geglu = self.fused_norm1 and (2 * c.ffn) * (c.d // 2) < 2 ** 31
        if self.fused_geglu:
            il = torch.arange(2 * c.ffn, device=self.dev).view(2, c.ffn).t().reshape(-1)
            self.wgu_il = [QWeightInt4G32(L["wgu"].packed.index_select(0, il).contiguous(),
                                          L["wgu"].scale.index_select(0, il).contiguous()) for L in weights["layers"]]
            if release_gate_up:
                for L in weights["layers"]:
                    del L["wgu"]
        # attention with the rotation and the cache write folded in, where its limits allow
        self.fused_attn = c.dh % 16 == 0 and c.max_ctx <= 65536
        if self.fused_attn:
            self.part = z(self.lib.chadq_attn_decode_mqa_fused_workspace_floats(c.hq, c.dh, c.max_ctx), f32)
            self.rope = z(c.max_ctx * c.dh, f32)
            _lib.check(self.lib.chadq_rope_table(self.rope.data_ptr(), c.dh, c.max_ctx, c.rope_base,
                                                 torch.cuda.current_stream().cuda_stream), "chadq_rope_table")
        else:
            self.part = z(self.lib.chadq_attn_decode_mqa_workspace_floats(c.hq, c.dh, c.max_ctx), f32)
        self.scratch = z(max(512, self.lib.chadq_gemv_i4g32_argmax_scratch_bytes(c.vocab, c.d) // 4), f32)
        self.token, self.pos = z(1, i32), z(1, i32)
        # sampling: (top_k, temperature) or None for greedy; the uniform draw lives in device memory, refreshed per step
        self.sampling = None
        self.u, self.sample_ws = z(1, f32), z(49152 // 4, f32)
        self.rng = torch.Generator(device=self.dev)
        self.kcache = [z(c.max_ctx * c.dh, bf16) for _ in range(c.n_layers)]
        self.vcache = [z(c.max_ctx * c.dh, bf16) for _ in range(c.n_layers)]
        self.graph = None
        self.graph_steps = 1        # tokens per replay of the captured graph
        self.ring = None            # the tokens between the steps of one replay (capture(steps > 1))

    # ---- single launches -------------------------------------------------------------------------------
    def _s(self):
        return torch.cuda.current_stream().cuda_stream

    def _gemv(self, x_bf16, qw: QWeightInt4G32, y):
        _lib.check(self.lib.chadq_gemv_i4g32(x_bf16.data_ptr(), qw.packed.data_ptr(), qw.scale.data_ptr(), y.data_ptr(),
                                             1, qw.N, qw.K, self._s()), "chadq_gemv_i4g32")

    def _norm(self, delta, w):
        nd = 0 if delta is None else delta.numel() // self.cfg.d
        _lib.check(self.lib.chadq_add_rmsnorm_bf16(self.x.data_ptr(), delta.data_ptr() if delta is not None else None, nd,
                                                   w.data_ptr(), self.xn.data_ptr(), self.cfg.d, self.cfg.eps, self._s()),
                   "chadq_add_rmsnorm_bf16")

    def embed_token(self) -> None:
        """self.x = the table row of self.token: what a step without its own embedding launch (step(embed=False), every
        step of a graph captured in greedy mode) expects to find.  A greedy step leaves the row of the token it chose
        there itself; call this after writing self.token by hand (set_state() does)."""
        c = self.cfg
        _lib.check(self.lib.chadq_embed_i4g32(self.token.data_ptr(), self.w["emb"].packed.data_ptr(), self.w["emb"].scale.data_ptr(),
                                              self.x.data_ptr(), c.d, c.vocab, self._s()), "chadq_embed_i4g32")

    def set_state(self, token: int, pos: int) -> None:
        """The token the next step consumes and its position, as feed() and generate() set them."""
        self._check_range(pos, 1, (token,))
        self.token.fill_(int(token))
        self.pos.fill_(int(pos))
        self.embed_token()

    def step(self, trace: Optional[list] = None, token_in=None, token_out=None, u=None, embed: bool = True) -> None:
        """One token: reads token/pos from device memory, leaves the next token and pos+1 there.  The caller keeps
        pos below max_ctx (feed() and generate() check it on the host; the kernels only clamp for memory safety).
        embed = False: self.x already holds the token's table row (embed_token(), or the greedy step before this one,
        whose last kernel writes the row of the token it chose), and the step saves the launch that would fetch it.
        trace (eager launches only, for parity checks): receives a copy of the fp32 residual vector entering every
        layer, then of the one entering the final norm (n_layers + 1 tensors).
        token_in / token_out / u (one-element device tensors; default self.token, self.token, self.u[:1]): where the
        step reads its token, leaves the next one and finds its uniform number - the steps of a multi-step graph
        hand their tokens on through a ring instead of through self.token."""
        c, lib, s = self.cfg, self.lib, self._s()
        token_in = self.token if token_in is None else token_in
        token_out = self.token if token_out is None else token_out
        u = self.u[:1] if u is None else u
        x_start = self.x  # the buffer a step starts from; the layers below may leave self.x naming the other one
        if embed:
            _lib.check(lib.chadq_embed_i4g32(token_in.data_ptr(), self.w["emb"].packed.data_ptr(), self.w["emb"].scale.data_ptr(),
                                             self.x.data_ptr(), c.d, c.vocab, s), "chadq_embed_i4g32")
        pending = None
        for li, L in enumerate(self.w["layers"]):
            if self.fused_norm1:
                nd = 0 if pending is None else pending.numel() // c.d
                _lib.check(lib.chadq_gemv_i4g32_addnorm(self.x.data_ptr(), pending.data_ptr() if nd else None, nd,
                                                        L["ln1"].data_ptr(), c.eps, self.x2.data_ptr(),
                                                        L["wqkv"].packed.data_ptr(), L["wqkv"].scale.data_ptr(),
                                                        self.qkv.data_ptr(), L["wqkv"].N, c.d, s), "chadq_gemv_i4g32_addnorm")
                self.x, self.x2 = self.x2, self.x  # the sum now lives in what was x2
            else:
                self._norm(pending, L["ln1"])
                self._gemv(self.xn, L["wqkv"], self.qkv)
            if trace is not None:
                trace.append(self.x.clone())  # the pending down projection has just been added: the layer's input
            if self.fused_attn and self.fused_oproj:
                _lib.check(lib.chadq_attn_decode_mqa_fused_oproj_i4g32(
                    self.qkv.data_ptr(), self.pos.data_ptr(), self.rope.data_ptr(), self.kcache[li].data_ptr(),
                    self.vcache[li].data_ptr(), self.part.data_ptr(), L["wo"].packed.data_ptr(), L["wo"].scale.data_ptr(),
                    self.ao.data_ptr(), c.hq, c.dh, c.max_ctx, c.d, s), "chadq_attn_decode_mqa_fused_oproj_i4g32")
            elif self.fused_attn:
                _lib.check(lib.chadq_attn_decode_mqa_fused(self.qkv.data_ptr(), self.pos.data_ptr(), self.rope.data_ptr(),
                                                           self.kcache[li].data_ptr(), self.vcache[li].data_ptr(),
                                                           self.part.data_ptr(), self.att.data_ptr(), c.hq, c.dh, c.max_ctx, s),
                           "chadq_attn_decode_mqa_fused")
            else:
                _lib.check(lib.chadq_rope_kv_write(self.qkv.data_ptr(), self.pos.data_ptr(), self.q.data_ptr(),
                                                   self.kcache[li].data_ptr(), self.vcache[li].data_ptr(), c.hq, c.dh,
                                                   c.max_ctx, c.rope_base, s), "chadq_rope_kv_write")
                _lib.check(lib.chadq_attn_decode_mqa(self.q.data_ptr(), self.kcache[li].data_ptr(), self.vcache[li].data_ptr(),
                                                     self.pos.data_ptr(), self.part.data_ptr(), self.att.data_ptr(), c.hq, c.dh,
                                                     c.max_ctx, s), "chadq_attn_decode_mqa")
            if not (self.fused_attn and self.fused_oproj):
                self._gemv(self.att, L["wo"], self.ao)
            nao = self.ao.numel() // c.d
            if self.fused_geglu:  # the second norm folds into the gate+up projection, the GeGLU into its epilogue
                wil = self.wgu_il[li]
                _lib.check(lib.chadq_gemv_i4g32_addnorm_geglu(self.x.data_ptr(), self.ao.data_ptr(), nao, L["ln2"].data_ptr(), c.eps,
                                                              self.x2.data_ptr(), wil.packed.data_ptr(), wil.scale.data_ptr(),
                                                              self.h.data_ptr(), wil.N, c.d, s), "chadq_gemv_i4g32_addnorm_geglu")
                self.x, self.x2 = self.x2, self.x
                if self.ksplit > 1:
                    _lib.check(lib.chadq_gemv_i4g32_splitk(self.h.data_ptr(), L["wd"].packed.data_ptr(), L["wd"].scale.data_ptr(),
                                                           self.dn.data_ptr(), c.d, c.ffn, self.ksplit, s), "chadq_gemv_i4g32_splitk")
                else:
                    self._gemv(self.h, L["wd"], self.dn)
                pending = self.dn
                continue
            self._norm(self.ao, L["ln2"])
            self._gemv(self.xn, L["wgu"], self.gu)
            if self.ksplit > 1:  # GeGLU folded into the split-K down projection
                _lib.check(lib.chadq_gemv_i4g32_splitk_geglu(self.gu.data_ptr(), L["wd"].packed.data_ptr(),
                                                             L["wd"].scale.data_ptr(), self.dn.data_ptr(), c.d, c.ffn,
                                                             self.ksplit, s), "chadq_gemv_i4g32_splitk_geglu")
            else:
                _lib.check(lib.chadq_geglu_bf16(self.gu.data_ptr(), self.h.data_ptr(), c.ffn, s), "chadq_geglu_bf16")
                self._gemv(self.h, L["wd"], self.dn)
            pending = self.dn
        self._norm(pending, self.w["lnf"])
        if trace is not None:
            trace.append(self.x.clone())
        if self.sampling is None:
            # the output table's GEMV leaves per-workgroup argmax candidates; the kernel that picks the winner also writes
            # the winner's table row where the next step starts from
            emb = self.w["emb"]
            _lib.check(lib.chadq_gemv_i4g32_argmax(self.xn.data_ptr(), emb.packed.data_ptr(), emb.scale.data_ptr(),
                                                   self.logits.data_ptr(), emb.N, emb.K, self.scratch.data_ptr(),
                                                   token_out.data_ptr(), self.pos.data_ptr(), 1, x_start.data_ptr(), s),
                       "chadq_gemv_i4g32_argmax")
        else:
            self._gemv(self.xn, self.w["emb"], self.logits)
            k, temperature = self.sampling
            _lib.check(lib.chadq_sample_topk_f32(self.logits.data_ptr(), c.vocab, k, temperature, u.data_ptr(),
                                                 self.sample_ws.data_ptr(), token_out.data_ptr(), self.pos.data_ptr(), 1, s),
                       "chadq_sample_topk_f32")
        if self.x is not x_start:  # an odd number of exchanges: the next step starts from the same buffer as this one
            self.x, self.x2 = x_start, self.x

    def set_sampling(self, top_k: int = 0, temperature: float = 1.0, seed: int = 0) -> None:
        """top_k = 0: greedy (argmax).  Otherwise the next token is drawn from the top_k most likely ones at the given
        temperature.  Call before capture(): a captured graph keeps the mode it was captured with."""
        if self.graph is not None:
            raise RuntimeError("set_sampling after capture(): the captured graph keeps its sampling mode")
        if top_k < 0 or top_k > min(64, self.cfg.vocab) or not temperature > 0:
            raise ValueError("top_k in 0..min(64, vocab) and temperature > 0 required")
        self.sampling = (int(top_k), float(temperature)) if top_k > 0 else None
        self.rng.manual_seed(seed)

    def _steps(self, k: int, embed_first: bool = True) -> None:
        """k consecutive steps; the token goes from one to the next through self.ring, in and out through self.token.
        Greedy steps hand the next token's table row on themselves: only the first may need a launch for it."""
        for j in range(k):
            self.step(token_in=self.token if j == 0 else self.ring[j:j + 1],
                      token_out=self.token if j == k - 1 else self.ring[j + 1:j + 2], u=self.u[j:j + 1],
                      embed=embed_first if j == 0 else self.sampling is not None)

    def capture(self, steps: int = 1) -> None:
        """Captures `steps` consecutive step() calls in one HIP graph (after an eager warm-up run whose effects are
        undone).  A replay then produces `steps` tokens: replaying a graph costs about 8 us over its nodes, once per
        replay.  The tokens of a replay are self.ring[1 : steps] followed by self.token; with sampling, step j of a
        replay draws with self.u[j].  feed() needs a one-step graph (or none): it sets the token before every step.
        A graph captured in greedy mode holds no embedding launch: it starts from the table row in self.x, which capture()
        itself, set_state(), feed(), generate() and every greedy step leave there; after writing self.token by hand,
        call embed_token() before the next replay."""
        if steps < 1 or steps > 64:
            raise ValueError("1 to 64 steps per graph")
        self.graph_steps = steps
        self.ring = torch.zeros(steps + 1, dtype=torch.int32, device=self.dev)
        if self.u.numel() < steps:
            self.u = torch.zeros(steps, dtype=torch.float32, device=self.dev)
        tok, pos = self.token.clone(), self.pos.clone()
        st = torch.cuda.Stream()
        st.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(st):
            self._steps(steps)
            torch.cuda.synchronize()
            self.token.copy_(tok)
            self.pos.copy_(pos)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=st):
                self._steps(steps, embed_first=self.sampling is not None)
            self.token.copy_(tok)
            self.pos.copy_(pos)
            self.embed_token()
        torch.cuda.current_stream().wait_stream(st)
        torch.cuda.synchronize()
        self.graph = g

    def _check_range(self, pos: int, n: int, tokens=()) -> None:
        """The kernels clamp a position to the cache and a token to the table so that nothing is addressed out of
        bounds, but a clamped step is a wrong step (it overwrites the last cache row and rotates by the wrong angle):
        refuse on the host what would run past the cache or name a token outside the vocabulary."""
        if pos < 0 or n < 0 or pos + n > self.cfg.max_ctx:
            raise ValueError("positions %d..%d do not fit the cache of %d rows" % (pos, pos + n - 1, self.cfg.max_ctx))
        for t in tokens:
            if not 0 <= int(t) < self.cfg.vocab:
                raise ValueError("token %d is outside the vocabulary [0, %d)" % (int(t), self.cfg.vocab))

    def feed(self, tokens, pos: int = 0) -> int:
        """Runs the step over a given token sequence starting at position `pos` (the prompt, one token at a time: there
        is no batched prefill here), filling the caches; returns the token the model proposes after the last one.
        Raises ValueError if the sequence would run past max_ctx or holds a token outside the vocabulary."""
        tokens = list(tokens)
        self._check_range(pos, len(tokens), tokens)
        self.pos.fill_(pos)
        for t in tokens:
            self.token.fill_(int(t))  # overrides the token the previous step proposed
            if self.sampling is not None:
                self.u.uniform_(0.0, 1.0, generator=self.rng)
            if self.graph is not None and self.graph_steps == 1:
                if self.sampling is None:
                    self.embed_token()  # a greedy graph starts from the row, and the row in place is the proposed token's
                self.graph.replay()
            else:
                self.step()
        return int(self.token.item())

    def generate(self, first_token: int, pos: int, n: int) -> List[int]:
        """Decodes n tokens starting from `first_token` at position `pos` (the cache holds pos rows): greedy, or sampled
        as set_sampling() says.  Raises ValueError if pos + n exceeds max_ctx or first_token is outside the vocabulary."""
        self._check_range(pos, n, (first_token,))
        self.token.fill_(first_token)
        self.pos.fill_(pos)
        self.embed_token()
        out = []
        k = self.graph_steps if self.graph is not None else 1
        while len(out) < n:
            if self.sampling is not None:
                self.u.uniform_(0.0, 1.0, generator=self.rng)  # eager, stream-ordered before the step or the replay
            if self.graph is not None and n - len(out) >= k:
                self.graph.replay()
                if k > 1:
                    out.extend(int(t) for t in torch.cat((self.ring[1:k], self.token)).tolist())
                    continue
            else:  # no graph, or fewer tokens left than a replay produces
                self.step()
            out.append(int(self.token.item()))
        return out
