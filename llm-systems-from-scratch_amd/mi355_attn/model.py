"""KV-cached inference model with the reference decoder's parameters and call surface.

`CachedTransformerLM` computes what TransformerLM.forward does (llm-core/llm_core/model.py:180-185:
embedding -> N x [RMSNorm -> causal attention with RoPE -> residual -> RMSNorm -> SwiGLU -> residual]
-> RMSNorm -> lm_head) from a reference `state_dict`, but keeps the K/V of every layer in a paged
cache, so that generation costs one prefill plus one single-token step per new token instead of the
reference's full forward over the whole context per token (model.py:218).

Device work: attention, RoPE + cache write, RMSNorm (with the residual add fused in) and
silu(gate)*up run on this package's HIP kernels; the projections are plain bf16 GEMMs
(`torch.matmul`, i.e. rocBLAS/hipBLASLt), with q/k/v and gate/up merged into one GEMM each
(the merge FusedSwiGLU makes, llm-systems/llm_systems/kernels/triton_swiglu.py:173-191).
Activations and weights are bf16, norm weights fp32.  There is no CPU path.
"""
from __future__ import annotations

import json

import torch

from . import ops
from .engine import BLOCK, PagedAttentionEngine


class CachedTransformerLM:
    def __init__(self, config: dict, state_dict: dict, *, num_blocks: int | None = None, max_batch: int = 64,
                 kv_dtype: str = "bf16", decode_graphs: bool = False, device="cuda:0"):
        """config: the reference's constructor arguments (model.py:128-137: vocab_size, context_length,
        d_model, num_layers, num_heads, d_ff, rope_theta); state_dict: the reference's parameter names,
        with either the separate (ffn.gate_proj/up_proj/down_proj) or the merged (ffn.w_gate_up/w_down)
        feed-forward weights.  num_blocks sizes the KV pool of every layer (default: max_batch full
        contexts); kv_dtype "fp8" keeps the pool as e4m3 bytes with per-(block, head) scales (half the
        cache bytes per decode step; d_head 64 or 128).  decode_graphs=True replays every decode step
        after the first of a batch size from a captured HIP graph (about ten launches per layer become one
        graph launch; the step's tensors then live at fixed addresses and tables have their full width)."""
        self.config = dict(config)
        self.device = torch.device(device)
        self.vocab_size = config["vocab_size"]
        self.context_length = config["context_length"]
        self.d_model = d = config["d_model"]
        self.num_layers = L = config["num_layers"]
        self.num_heads = H = config["num_heads"]
        self.d_ff = config["d_ff"]
        if d % H:
            raise ValueError("d_model must be divisible by num_heads")
        self.d_head = d // H
        if self.d_head not in (32, 64, 128):
            raise ValueError("the attention kernels need d_head in {32, 64, 128}")
        sd = {k[len("_orig_mod."):] if k.startswith("_orig_mod.") else k: v for k, v in state_dict.items()}  # model.py:247-251

        def w(name, dtype=torch.bfloat16):
            return sd[name].detach().to(device=self.device, dtype=dtype).contiguous()

        self.emb = w("token_embeddings.weight")
        self.lm_head = w("lm_head.weight")
        self.final_norm = w("final_norm.weight", torch.float32)
        self.layers = []
        for i in range(L):
            pre = f"layers.{i}."
            wqkv = torch.cat([w(pre + f"attn.{n}.weight") for n in ("q_proj", "k_proj", "v_proj")])
            if pre + "ffn.w_gate_up.weight" in sd:
                wgu, wdown = w(pre + "ffn.w_gate_up.weight"), w(pre + "ffn.w_down.weight")
            else:
                wgu = torch.cat([w(pre + "ffn.gate_proj.weight"), w(pre + "ffn.up_proj.weight")])
                wdown = w(pre + "ffn.down_proj.weight")
            self.layers.append(dict(wqkv=wqkv, wo=w(pre + "attn.output_proj.weight"), wgu=wgu, wdown=wdown,
                                    attn_norm=w(pre + "attn_norm.weight", torch.float32),
                                    ffn_norm=w(pre + "ffn_norm.weight", torch.float32)))
        if num_blocks is None:
            num_blocks = max_batch * ((self.context_length + BLOCK - 1) // BLOCK)
        self.engine = PagedAttentionEngine(num_blocks, H, H, self.d_head, self.context_length,
                                           rope_theta=config["rope_theta"], max_batch=max_batch, num_layers=L,
                                           kv_dtype=kv_dtype, device=self.device)
        self._next_id = 0
        self.decode_graphs = decode_graphs
        self._graphs = {}                      # batch size -> [static step tensors, captured graph, its logits]

    @classmethod
    def from_pretrained(cls, config_path: str, checkpoint_path: str, **kwargs) -> "CachedTransformerLM":
        """Same files as TransformerLM.from_pretrained (model.py:238-256): a JSON config and a checkpoint that is
        a state_dict or {"model": state_dict}.  The checkpoint is read with weights_only=True."""
        with open(config_path) as f:
            config = json.load(f)
        sd = torch.load(checkpoint_path, map_location="cpu", weights_only=True)
        if "model" in sd:
            sd = sd["model"]
        return cls(config, sd, **kwargs)

    # ---- the decoder on packed tokens ------------------------------------------------------
    def _forward(self, token_ids, plan, attend, out_rows=None):
        """token_ids (T,) int64 on the device; attend(layer, plan, q, k, v) -> (T,H,d_head).
        Returns logits of rows `out_rows` (default: all rows), fp32."""
        H, dh, d, ff = self.num_heads, self.d_head, self.d_model, self.d_ff
        T = token_ids.shape[0]
        resid = self.emb[token_ids]                                   # model.py:50
        h = ops.rms_norm(resid, self.layers[0]["attn_norm"])
        for i, ly in enumerate(self.layers):
            qkv = (h @ ly["wqkv"].T).view(T, 3, H, dh)                 # model.py:361-370 in one GEMM
            a = attend(i, plan, qkv[:, 0], qkv[:, 1], qkv[:, 2])      # model.py:372-385
            o = a.reshape(T, d) @ ly["wo"].T                           # model.py:388-390
            h, resid = ops.rms_norm(o, ly["ffn_norm"], residual=resid, return_sum=True)    # model.py:293-294
            gu = h @ ly["wgu"].T
            f = ops.silu_mul(gu[:, :ff], gu[:, ff:]) @ ly["wdown"].T   # model.py:304-305
            nxt = self.layers[i + 1]["attn_norm"] if i + 1 < self.num_layers else self.final_norm
            h, resid = ops.rms_norm(f, nxt, residual=resid, return_sum=True)              # model.py:294, :184
        if out_rows is not None:
            h = h[out_rows]
        return (h @ self.lm_head.T).float()                            # model.py:185

    # ---- sequence-level API ---------------------------------------------------------------------
    def new_sequence(self) -> int:
        sid = self._next_id
        self._next_id += 1
        self.engine.add_sequence(sid)
        return sid

    def free_sequence(self, seq_id: int) -> None:
        self.engine.remove_sequence(seq_id)

    def prefill(self, seq_ids, prompts, *, all_logits: bool = False):
        """Runs the prompts (lists / 1-D tensors of token ids, each 1..context_length long) of new sequences.
        Returns next-token logits (n_seq, vocab) fp32, or the logits of every prompt position
        (sum(len), vocab) with all_logits=True."""
        toks = [torch.as_tensor(p, dtype=torch.int64).reshape(-1) for p in prompts]
        plan = self.engine.plan_prefill(list(seq_ids), [int(t.numel()) for t in toks])
        ids = torch.cat(toks).to(self.device)
        return self._forward(ids, plan, self.engine.attend_prefill, None if all_logits else plan.last_rows)

    def decode(self, seq_ids, tokens):
        """Appends one token to each running sequence; returns the next-token logits (n_seq, vocab) fp32."""
        seq_ids = list(seq_ids)
        if self.decode_graphs:
            return self._decode_graphed(seq_ids, torch.as_tensor(tokens).reshape(-1).tolist())
        ids = torch.as_tensor(tokens, dtype=torch.int64).reshape(-1).to(self.device)
        if ids.numel() != len(seq_ids):
            raise ValueError("one token per sequence expected")
        plan = self.engine.plan_decode(seq_ids)
        return self._forward(ids, plan, self.engine.attend_decode)

    def _decode_graphed(self, seq_ids, tokens):
        """The decode step through a HIP graph.  The first step of a batch size runs eagerly on the static
        step tensors (which also initialises every library the graph will call) and is then captured; later
        steps refresh the static tensors with one copy and replay."""
        B = len(seq_ids)
        if len(tokens) != B:
            raise ValueError("one token per sequence expected")
        entry = self._graphs.get(B)
        if entry is None:
            entry = self._graphs[B] = [self.engine.make_static_decode(B), None, None]
        static = entry[0]
        plan = self.engine.plan_decode_into(seq_ids, tokens, static)
        if entry[1] is None:
            logits = self._forward(static.tokens, plan, self.engine.attend_decode)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                entry[2] = self._forward(static.tokens, plan, self.engine.attend_decode)
            entry[1] = graph
            return logits
        entry[1].replay()
        return entry[2].clone()

    def forward(self, token_ids):
        """Logits (batch, seq, vocab) of whole sequences, as TransformerLM.forward returns them
        (model.py:180-185); nothing stays in the cache afterwards."""
        token_ids = torch.as_tensor(token_ids)
        if token_ids.dim() == 1:
            token_ids = token_ids[None]
        Bn, S = token_ids.shape
        sids = [self.new_sequence() for _ in range(Bn)]
        try:
            logits = self.prefill(sids, list(token_ids), all_logits=True)
        finally:
            for s in sids:
                self.free_sequence(s)
        return logits.view(Bn, S, self.vocab_size)

    # ---- sampling loops -----------------------------------------------------------------------------
    @staticmethod
    def _sample(logits, temperature, top_k, generator=None):
        """model.py:219-228.  temperature 0 means argmax.  top_k keeps the k largest logits -- what the
        reference's :221-225 is written to do (its masked_fill result is discarded, so the reference itself
        samples from all tokens whatever top_k says)."""
        if temperature == 0:
            return logits.argmax(-1, keepdim=True)
        scaled = logits / temperature
        if top_k:
            kth = torch.topk(scaled, min(top_k, scaled.size(-1))).values[:, -1:]
            scaled = scaled.masked_fill(scaled < kth, float("-inf"))
        return torch.multinomial(torch.softmax(scaled, dim=-1), 1, generator=generator)

    @torch.no_grad()
    def generate(self, prompt_ids, max_new_tokens: int, temperature: float = 1.0, top_k: int | None = None,
                 eos_token_id: int | None = None, *, generator=None):
        """Same arguments and result as TransformerLM.generate (model.py:187-236): prompt (1, seq) or (seq,),
        returns the generated ids (1, n), stopping before an eos token.  Once prompt + generated tokens exceed
        context_length the reference re-encodes the last context_length tokens from position 0 on every step
        (:215); this does the same by re-running the prefill over that window (no cache reuse is possible
        there, the positions of all cached keys change)."""
        ids = [int(t) for t in torch.as_tensor(prompt_ids).reshape(-1).tolist()]
        if not ids:
            raise ValueError("empty prompt")
        out = []
        sid = self.new_sequence()
        try:
            logits = self.prefill([sid], [ids[-self.context_length:]])
            for step in range(max_new_tokens):
                nxt = int(self._sample(logits, temperature, top_k, generator).item())
                if eos_token_id is not None and nxt == eos_token_id:
                    break
                ids.append(nxt)
                out.append(nxt)
                if step + 1 == max_new_tokens:
                    break
                if self.engine.lengths[sid] < self.context_length:
                    logits = self.decode([sid], [nxt])
                else:                                   # window slides: positions restart at 0 (model.py:215)
                    self.free_sequence(sid)
                    sid = self.new_sequence()
                    logits = self.prefill([sid], [ids[-self.context_length:]])
        finally:
            self.free_sequence(sid)
        return torch.tensor([out], dtype=torch.int64, device=self.device)

    @torch.no_grad()
    def generate_batch(self, prompts, max_new_tokens: int, temperature: float = 1.0, top_k: int | None = None,
                       eos_token_id: int | None = None, *, generator=None):
        """Continuous batching: all prompts are prefilled in one packed pass, then every step decodes one token
        for each sequence still running (finished ones leave the batch and free their blocks).  A sequence also
        stops when it fills its context.  Returns a list of token lists."""
        n = len(prompts)
        if n > self.engine.max_batch:
            raise ValueError(f"{n} prompts exceed max_batch {self.engine.max_batch}")
        sids = [self.new_sequence() for _ in range(n)]
        outs = [[] for _ in range(n)]
        live = list(range(n))
        try:
            logits = self.prefill(sids, prompts)
            for step in range(max_new_tokens):
                nxt = self._sample(logits, temperature, top_k, generator).reshape(-1).tolist()
                keep, toks = [], []
                for j, i in enumerate(live):
                    t = int(nxt[j])
                    if eos_token_id is not None and t == eos_token_id:
                        continue
                    outs[i].append(t)
                    if self.engine.lengths[sids[i]] < self.context_length:
                        keep.append(i)
                        toks.append(t)
                for i in live:
                    if i not in keep:
                        self.free_sequence(sids[i])
                        sids[i] = None
                live = keep
                if not live or step + 1 == max_new_tokens:
                    break
                logits = self.decode([sids[i] for i in live], toks)
        finally:
            for s in sids:
                if s is not None and s in self.engine.blocks:
                    self.free_sequence(s)
        return outs
