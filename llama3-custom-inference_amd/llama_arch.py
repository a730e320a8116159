"""Llama-3 architecture harness around the three custom operators, for the end-to-end
measurement (random-init weights, synthetic prompts, greedy decode).

It reproduces how the reference's model.py drives the operators -- the four call sites with
the same tensor layouts and views -- without its checkpoint loading:

  RMSNorm.forward                model.py:70-72     -> ops.rms_norm(x, weight, eps)
  CausalSelfAttention.forward    model.py:92-122    -> ops.rot_embed(q|k views of the fused qkv
                                                       projection, freqs), static KV cache
                                                       (maxB, L, KVH, HD) sliced and transposed,
                                                       ops.flash_attention_decode(q, k, v) when T == 1,
                                                       ops.flash_attention_prefill (or torch SDPA) for the prefill
  LLaMA3.forward                 model.py:203-232   -> embedding, blocks, final norm, tied lm_head
                                                       on the last position, float32 logits
  LLaMA3.generate                model.py:313-396   -> prompt mask keep, argmax when temperature is 0,
                                                       stop-token bookkeeping with one device-side .all()
                                                       (the reference iterates the tensor in Python, :380)

Embedding, sampling and every nn.Linear with more than a few activation rows stay stock PyTorch,
as in the reference; the linears of the decode step (T == 1) use ops.linear_decode /
ops.linear_swiglu_decode when the operator module has them.  `ops` is the
module that provides the three operators: custom_kernels.custom_kernels_extension on the GPU,
or any object with the same three functions (the CPU baseline passes torch restatements).
"""

import math
import time
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from custom_kernels import precompute_freqs_cis


@dataclass
class LlamaConfig:
    """Hyper-parameters with the reference's names and Llama-3.2-1B defaults (model.py:153-166)."""
    block_size: int = 8192
    vocab_size: int = 128256
    n_layer: int = 16
    n_head: int = 32
    n_kv_head: int = 8
    n_embd: int = 2048
    hidden_dim: int = 8192
    norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    use_scaled_rope: bool = True
    rope_scale_factor: float = 32.0   # model.py:29 hard-codes 8 (Llama-3.1); Llama-3.2 uses 32
    max_model_len: int = 256
    max_gen_batch_size: int = 256

    def __post_init__(self):
        assert self.n_kv_head <= self.n_head and self.n_head % self.n_kv_head == 0
        assert self.n_embd % self.n_head == 0


class _Tokenizer:
    """Stand-in carrying what generate() reads from the HF tokenizer (model.py:307-308)."""
    pad_id = 128004
    stop_tokens = (128001,)


class LlamaDecoder:
    MAX_DECODE_LOOPS = 8    # (batch, total length) pairs whose recorded decode loops are kept

    def __init__(self, config: LlamaConfig, ops, device, dtype=torch.bfloat16, seed: int = 42, weights_from=None):
        """`weights_from`: another LlamaDecoder of the same configuration whose weights are copied
        (to this device) instead of being drawn again from the seed."""
        self.config, self.ops, self.device, self.dtype = config, ops, torch.device(device), dtype
        self.tokenizer = _Tokenizer()
        c = config
        hd = c.n_embd // c.n_head
        self.hd = hd
        g = torch.Generator().manual_seed(seed)
        donor = iter(weights_from._weights()) if weights_from is not None else None

        def w(*shape):
            if donor is not None:
                t = next(donor)
                assert tuple(t.shape) == tuple(shape)
                return t.to(device=self.device, dtype=dtype)
            return (torch.randn(shape, generator=g, dtype=torch.float32) * 0.02).to(dtype).to(self.device)

        self.wte = w(c.vocab_size, c.n_embd)          # tied with the lm_head (model.py:190)
        self.layers = []
        for _ in range(c.n_layer):
            self.layers.append(dict(
                ln_1=torch.ones(c.n_embd, dtype=dtype, device=self.device),
                c_attn=w((c.n_head + 2 * c.n_kv_head) * hd, c.n_embd),
                c_proj=w(c.n_embd, c.n_embd),
                ln_2=torch.ones(c.n_embd, dtype=dtype, device=self.device),
                c_fc=w(c.hidden_dim, c.n_embd),
                c_fc2=w(c.hidden_dim, c.n_embd),
                mlp_proj=w(c.n_embd, c.hidden_dim),
                cache_k=torch.zeros((c.max_gen_batch_size, c.max_model_len, c.n_kv_head, hd), dtype=dtype,
                                    device=self.device),
                cache_v=torch.zeros((c.max_gen_batch_size, c.max_model_len, c.n_kv_head, hd), dtype=dtype,
                                    device=self.device),
            ))
        self.ln_f = torch.ones(c.n_embd, dtype=dtype, device=self.device)
        self.freqs_cis = precompute_freqs_cis(hd, c.block_size * 2, c.rope_theta, c.use_scaled_rope,
                                              scale_factor=c.rope_scale_factor, device=self.device)
        self.prefill_backend = "unset"
        self._graphs = {}
        # nn.Linear calls with at most this many activation rows (the decode step) go through the
        # library's weight-streaming kernels when the operator module has them; 0 = always F.linear
        self.decode_linear_rows = 16 if hasattr(ops, "linear_decode") else 0

    def _weights(self):
        """The random-init matrices in the order __init__ draws them."""
        yield self.wte
        for L in self.layers:
            for name in ("c_attn", "c_proj", "c_fc", "c_fc2", "mlp_proj"):
                yield L[name]

    def prefill_pass_mode(self):
        """How generate_graphed ran its prompt passes so far: 'recorded' (HIP graph, checked against the
        eager pass), 'eager' (the recording did not reproduce the eager logits) or 'none yet'."""
        entries = [e for loop in self._graphs.values() for e in loop.prefill_graphs.values()]
        if not entries:
            return "none yet"
        return "recorded" if all(e[0] is not None for e in entries) else "eager"

    def set_decode_linear_rows(self, rows: int):
        self.decode_linear_rows = rows if hasattr(self.ops, "linear_decode") else 0
        self._graphs.clear()   # recorded decode steps contain the previous choice

    def _linear(self, x, w):
        """x @ w.T (nn.Linear without bias: model.py:95,121,134,225)."""
        if 0 < x.numel() // x.shape[-1] <= self.decode_linear_rows:
            return self.ops.linear_decode(x, w)
        return F.linear(x, w)

    def _mlp(self, L, h):
        """c_proj(silu(c_fc2(h)) * c_fc(h)) (model.py:134)."""
        if 0 < h.numel() // h.shape[-1] <= self.decode_linear_rows:
            return self.ops.linear_decode(self.ops.linear_swiglu_decode(h, L["c_fc2"], L["c_fc"]), L["mlp_proj"])
        return F.linear(F.silu(F.linear(h, L["c_fc2"])) * F.linear(h, L["c_fc"]), L["mlp_proj"])

    # ------------------------------------------------------------------ attention block
    def _attention(self, L, x, freqs_cis, start_pos):
        y = self._attention_core(L, self._linear(x, L["c_attn"]), freqs_cis, start_pos)
        return self._linear(y, L["c_proj"])

    def _attention_core(self, L, qkv, freqs_cis, start_pos):
        """From the fused qkv projection to the attention output (B, T, C), before c_proj."""
        c = self.config
        B, T = qkv.shape[:2]
        hd = self.hd
        q, k, v = qkv.split([c.n_head * hd, c.n_kv_head * hd, c.n_kv_head * hd], dim=-1)
        q, k, v = (t.view(B, T, -1, hd) for t in (q, k, v))        # strided views into qkv
        q = self.ops.rot_embed(q, freqs_cis)
        k = self.ops.rot_embed(k, freqs_cis)
        L["cache_k"][:B, start_pos:start_pos + T] = k
        L["cache_v"][:B, start_pos:start_pos + T] = v
        k = L["cache_k"][:B, :start_pos + T]
        v = L["cache_v"][:B, :start_pos + T]
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))           # (B, H, T|S, HD) views
        if T > 1:
            y = self._prefill_attention(q, k, v)
        else:
            y = self.ops.flash_attention_decode(q, k, v)
        return y.transpose(1, 2).contiguous().view(B, T, c.n_embd)

    FUSED_MAX_ROWS = 4   # rows up to which the fused single-launch linears carry the whole decode step
    QKV_FUSED_MAX_ROWS = 16   # rows up to which the split-K route takes the single-launch qkv + rope + append linear (+2..6 %)
    SWIGLU_MAX_ROWS = 14  # rows up to which the split-K route takes the single-launch gate|up + SwiGLU linear (+3 % at 7..10 rows, level at 16)

    def _splitk(self, rows: int) -> bool:
        """5..64 activation rows: the split-K linears (activations shared through LDS, splits added
        up by the operator that follows) stand for F.linear on the output and down projections, and
        from 17 rows on for the qkv projection too.  Measured end to end, this route overtakes the
        fused single-launch linears at 5 rows (+6 % at 5, +8 % at 6, more beyond): every workgroup of
        those re-reads the activations of its k range, which the 8192-wide down projection feels first."""
        return self.decode_linear_rows > 0 and self.FUSED_MAX_ROWS < rows <= 64 and hasattr(self.ops, "linear_splitk")

    def _gate_up(self, L):
        """c_fc2 and c_fc stacked into one (2 * hidden, C) matrix: one GEMM instead of two."""
        if "c_fc_cat" not in L:
            L["c_fc_cat"] = torch.cat([L["c_fc2"], L["c_fc"]], dim=0)
        return L["c_fc_cat"]

    def _decode_layers_splitk(self, x, append_and_attend, project_and_attend=None):
        """The layers of one decode step (T == 1) at 5..64 rows; returns the final hidden state.
        append_and_attend(L, qkv partial products) -> attention output (B, 1, C);
        project_and_attend(L, normalised input) -> the same from the single-launch qkv projection
        (rotary embedding and cache append inside), taken while the rows are few enough for it."""
        c, ops = self.config, self.ops
        H = c.hidden_dim
        rows = x.numel() // x.shape[-1]
        qkv_fused = project_and_attend is not None and rows <= self.QKV_FUSED_MAX_ROWS
        h = ops.rms_norm(x, self.layers[0]["ln_1"], c.norm_eps)
        for i, L in enumerate(self.layers):
            y = project_and_attend(L, h) if qkv_fused else append_and_attend(L, ops.linear_splitk(h, L["c_attn"]))
            x, h = ops.add_rms_norm_partials(x, ops.linear_splitk(y, L["c_proj"]), L["ln_2"], c.norm_eps)
            if rows <= self.SWIGLU_MAX_ROWS:
                t = ops.linear_swiglu_decode(h, L["c_fc2"], L["c_fc"])     # one launch for the pair and the product
            else:
                gu = F.linear(h, self._gate_up(L))
                t = ops.silu_mul(gu[..., :H], gu[..., H:])
            next_norm = self.layers[i + 1]["ln_1"] if i + 1 < len(self.layers) else self.ln_f
            x, h = ops.add_rms_norm_partials(x, ops.linear_splitk(t, L["mlp_proj"]), next_norm, c.norm_eps)
        return h

    def _fused_rows(self) -> int:
        """Rows up to which the decode step uses linear_decode_fused (norms and residual additions
        folded into the linears); 0 when the operator module has no such operator."""
        f = getattr(self.ops, "linear_decode_fused_max_rows", None)
        return min(self.decode_linear_rows, f(self.config.n_embd), self.FUSED_MAX_ROWS) if f else 0

    def _prefill_attention(self, q, k, v):
        """Causal GQA attention for T > 1.  The reference hands this case to torch
        (model.py:114-116); here it goes through the library's prefill kernel when the operator
        module provides one (the CPU stand-in does not and uses torch, like the reference)."""
        op = getattr(self.ops, "flash_attention_prefill", None)
        if op is not None:
            self.prefill_backend = "l3 prefill kernel"
            return op(q, k, v)
        self.prefill_backend = "torch.sdpa"
        return F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)

    def forward(self, idx, start_pos=0):
        """idx (B, T) token ids -> float32 logits (B, 1, vocab) of the last position."""
        c = self.config
        B, T = idx.shape
        assert T <= c.block_size
        x = F.embedding(idx, self.wte)
        freqs_cis = self.freqs_cis[start_pos:start_pos + T]
        if T == 1 and 0 < B <= self._fused_rows():
            # decode step with the norms and residual additions folded into the linears
            lin = self.ops.linear_decode_fused
            for L in self.layers:
                qkv = lin(x, L["c_attn"], norm_weight=L["ln_1"], eps=c.norm_eps)
                x = lin(self._attention_core(L, qkv, freqs_cis, start_pos), L["c_proj"], residual=x)
                t = lin(x, L["c_fc2"], norm_weight=L["ln_2"], eps=c.norm_eps, w_up=L["c_fc"])
                x = lin(t, L["mlp_proj"], residual=x)
            return lin(x, self.wte, norm_weight=self.ln_f, eps=c.norm_eps).float()
        if T == 1 and self._splitk(B):
            pos = torch.tensor([start_pos], dtype=torch.int32, device=self.device)

            def append_and_attend(L, part):
                q = self.ops.rot_embed_append_partials(part, self.freqs_cis, L["cache_k"], L["cache_v"], pos, c.n_head)
                y = self.ops.flash_attention_decode(q.transpose(1, 2), L["cache_k"][:B, :start_pos + 1].transpose(1, 2),
                                                    L["cache_v"][:B, :start_pos + 1].transpose(1, 2))
                return y.transpose(1, 2).reshape(B, 1, c.n_embd)

            def project_and_attend(L, hn):
                q = self.ops.linear_qkv_rope_append(hn, L["c_attn"], self.freqs_cis, L["cache_k"], L["cache_v"], pos,
                                                    c.n_head)
                y = self.ops.flash_attention_decode(q.transpose(1, 2), L["cache_k"][:B, :start_pos + 1].transpose(1, 2),
                                                    L["cache_v"][:B, :start_pos + 1].transpose(1, 2))
                return y.transpose(1, 2).reshape(B, 1, c.n_embd)

            h = self._decode_layers_splitk(x, append_and_attend, project_and_attend)
            return F.linear(h, self.wte).float()
        for L in self.layers:
            x = x + self._attention(L, self.ops.rms_norm(x, L["ln_1"], c.norm_eps), freqs_cis, start_pos)
            h = self.ops.rms_norm(x, L["ln_2"], c.norm_eps)
            x = x + self._mlp(L, h)
        x = self.ops.rms_norm(x, self.ln_f, c.norm_eps)
        return self._linear(x[:, -1:, :].contiguous(), self.wte).float()

    # ------------------------------------------------------------------------- generate
    @torch.inference_mode()
    def generate_graphed(self, prompt_tokens, max_gen_len, echo=False, ignore_eos=False):
        """generate() with the per-token loop replayed from a HIP graph: the prefill of the common
        prompt prefix (model.py:365 with T = min_prompt_len) is one recorded pass, every later position
        one replay of the recorded decode step.  Needs ops with rot_embed_append / flash_attention_decode_devlen."""
        c = self.config
        bsz = len(prompt_tokens)
        min_prompt_len = min(len(t) for t in prompt_tokens)
        max_prompt_len = max(len(t) for t in prompt_tokens)
        total_len = min(c.block_size, max_gen_len + max_prompt_len)
        assert bsz <= c.max_gen_batch_size and total_len <= c.max_model_len
        key = (bsz, total_len)
        loop = self._graphs.get(key)
        if loop is None:
            while len(self._graphs) >= self.MAX_DECODE_LOOPS:      # recorded loops hold device memory
                self._graphs.pop(next(iter(self._graphs)))
            loop = GraphedDecodeLoop(self, bsz, total_len)
            self._graphs[key] = loop
        pad_id = self.tokenizer.pad_id
        host = torch.full((bsz, total_len), pad_id, dtype=torch.long)
        for i, t in enumerate(prompt_tokens):
            host[i, :len(t)] = torch.tensor(t, dtype=torch.long)
        loop.tokens.copy_(host)
        loop.text_mask.copy_(host != pad_id)
        loop.eos.zero_()
        # position min_prompt_len: prefill (recorded once per prompt length) + the usual bookkeeping
        logits = loop.prefill(self, min_prompt_len)
        nxt = torch.argmax(logits[:, -1], dim=-1)
        if min_prompt_len < total_len:
            keep = loop.text_mask[:, min_prompt_len]
            nxt = torch.where(keep, loop.tokens[:, min_prompt_len], nxt)
            loop.tokens[:, min_prompt_len] = nxt
            loop.eos |= ~keep & torch.isin(nxt, loop.stop)
        loop.tok.copy_(nxt.unsqueeze(1))
        loop.pos.fill_(min_prompt_len)
        loop.kv_len.fill_(min_prompt_len + 1)
        if loop.graph is None:
            loop.capture(self)
        for cur_pos in range(min_prompt_len + 1, total_len):
            loop.graph.replay()
            if not ignore_eos and (cur_pos - min_prompt_len) % 16 == 0 and bool(loop.eos.all()):
                break
        out = []
        for i, toks in enumerate(loop.tokens.tolist()):
            start = 0 if echo else len(prompt_tokens[i])
            toks = toks[start:len(prompt_tokens[i]) + max_gen_len]
            for s_ in self.tokenizer.stop_tokens:
                if s_ in toks and not ignore_eos:
                    toks = toks[:toks.index(s_)]
            out.append(toks)
        return out

    @torch.inference_mode()
    def generate(self, prompt_tokens, max_gen_len, temperature=0.0, echo=False, ignore_eos=False):
        """Greedy (temperature 0) generation with the reference's bookkeeping (model.py:340-396);
        sampling is out of scope here and raises."""
        if temperature > 0:
            raise NotImplementedError("the harness measures greedy decode (temperature 0)")
        c = self.config
        bsz = len(prompt_tokens)
        assert bsz <= c.max_gen_batch_size
        min_prompt_len = min(len(t) for t in prompt_tokens)
        max_prompt_len = max(len(t) for t in prompt_tokens)
        assert max_prompt_len <= c.block_size
        total_len = min(c.block_size, max_gen_len + max_prompt_len)
        assert total_len <= c.max_model_len, "KV cache too short for prompt + generation"
        pad_id = self.tokenizer.pad_id
        tokens = torch.full((bsz, total_len), pad_id, dtype=torch.long, device=self.device)
        for i, t in enumerate(prompt_tokens):
            tokens[i, :len(t)] = torch.tensor(t, dtype=torch.long, device=self.device)
        input_text_mask = tokens != pad_id
        stop_tokens = torch.tensor(list(self.tokenizer.stop_tokens), device=self.device)
        eos_reached = torch.zeros(bsz, dtype=torch.bool, device=self.device)
        prev_pos = 0
        for cur_pos in range(min_prompt_len, total_len):
            logits = self.forward(tokens[:, prev_pos:cur_pos], start_pos=prev_pos)
            next_token = torch.argmax(logits[:, -1], dim=-1).reshape(-1)
            next_token = torch.where(input_text_mask[:, cur_pos], tokens[:, cur_pos], next_token)
            tokens[:, cur_pos] = next_token
            eos_reached |= ~input_text_mask[:, cur_pos] & torch.isin(next_token, stop_tokens)
            prev_pos = cur_pos
            if not ignore_eos and bool(eos_reached.all()):
                break
        out = []
        for i, toks in enumerate(tokens.tolist()):
            start = 0 if echo else len(prompt_tokens[i])
            toks = toks[start:len(prompt_tokens[i]) + max_gen_len]
            for s in self.tokenizer.stop_tokens:
                if s in toks and not ignore_eos:
                    toks = toks[:toks.index(s)]
            out.append(toks)
        return out


class GraphedDecodeLoop:
    """The single-token decode step of LlamaDecoder recorded once as a HIP graph and replayed per
    generated token (the reference's loop, model.py:363-381, launches ~450 kernels per token from
    Python; at batch 1 that, not the GPU, sets the pace).

    What makes the step replayable: the token position lives in device memory.  The fused
    rot_embed_append operator writes K/V at that position, flash_attention_decode_devlen reads the
    KV length from it, residual additions ride along with the norms (add_rms_norm), and the bookkeeping of generate() (prompt-mask keep, token store, stop
    flags, position increment) is expressed with fixed-shape torch ops on device tensors.
    """

    def __init__(self, model: "LlamaDecoder", batch: int, total_len: int):
        import torch as _t

        # The loop does not keep the model: the model owns its loops (LlamaDecoder._graphs), and a
        # reference cycle would leave the recorded graph to the cyclic garbage collector, which may
        # then destroy it in the middle of another stream capture (that aborts the process).
        self.B, self.total_len = batch, total_len
        dev = model.device
        self.tokens = _t.zeros((batch, total_len), dtype=_t.long, device=dev)
        self.text_mask = _t.zeros((batch, total_len), dtype=_t.bool, device=dev)
        self.tok = _t.zeros((batch, 1), dtype=_t.long, device=dev)     # token fed to this step
        self.pos = _t.zeros(1, dtype=_t.int32, device=dev)             # its position = cache row written
        self.kv_len = _t.ones(1, dtype=_t.int32, device=dev)           # pos + 1
        self.eos = _t.zeros(batch, dtype=_t.bool, device=dev)
        self.stop = _t.tensor(list(model.tokenizer.stop_tokens), device=dev)
        self.graph = None
        self.prefill_graphs = {}   # prompt length -> (recorded prefill or None when it failed its check, logits)

    def step(self, m: "LlamaDecoder"):
        c, B = m.config, self.B
        ops = m.ops
        x = F.embedding(self.tok, m.wte)
        if 0 < B <= m._fused_rows():
            # five launches per layer: norms, rotary embedding, cache append and residual additions ride
            # with the linears
            lin = ops.linear_decode_fused
            for L in m.layers:
                q = ops.linear_qkv_rope_append(x, L["c_attn"], m.freqs_cis, L["cache_k"], L["cache_v"], self.pos,
                                               c.n_head, norm_weight=L["ln_1"], eps=c.norm_eps)
                y = ops.flash_attention_decode_devlen(q.transpose(1, 2), L["cache_k"][:B].transpose(1, 2),
                                                      L["cache_v"][:B].transpose(1, 2), self.kv_len)
                x = lin(y.transpose(1, 2).reshape(B, 1, c.n_embd), L["c_proj"], residual=x)
                t = lin(x, L["c_fc2"], norm_weight=L["ln_2"], eps=c.norm_eps, w_up=L["c_fc"])
                x = lin(t, L["mlp_proj"], residual=x)
            logits = lin(x[:, -1], m.wte, norm_weight=m.ln_f, eps=c.norm_eps)
        elif m._splitk(B):
            def append_and_attend(L, part):
                q = ops.rot_embed_append_partials(part, m.freqs_cis, L["cache_k"], L["cache_v"], self.pos, c.n_head)
                y = ops.flash_attention_decode_devlen(q.transpose(1, 2), L["cache_k"][:B].transpose(1, 2),
                                                      L["cache_v"][:B].transpose(1, 2), self.kv_len)
                return y.transpose(1, 2).reshape(B, 1, c.n_embd)

            def project_and_attend(L, hn):
                q = ops.linear_qkv_rope_append(hn, L["c_attn"], m.freqs_cis, L["cache_k"], L["cache_v"], self.pos,
                                               c.n_head)
                y = ops.flash_attention_decode_devlen(q.transpose(1, 2), L["cache_k"][:B].transpose(1, 2),
                                                      L["cache_v"][:B].transpose(1, 2), self.kv_len)
                return y.transpose(1, 2).reshape(B, 1, c.n_embd)

            logits = F.linear(m._decode_layers_splitk(x, append_and_attend, project_and_attend)[:, -1], m.wte)
        else:
            h = ops.rms_norm(x, m.layers[0]["ln_1"], c.norm_eps)
            for i, L in enumerate(m.layers):
                qkv = m._linear(h, L["c_attn"])
                q = ops.rot_embed_append(qkv, m.freqs_cis, L["cache_k"], L["cache_v"], self.pos, c.n_head)
                y = ops.flash_attention_decode_devlen(q.transpose(1, 2), L["cache_k"][:B].transpose(1, 2),
                                                      L["cache_v"][:B].transpose(1, 2), self.kv_len)
                # residual add fused with the norm that follows it (same bits as add, then rms_norm)
                x, h = ops.add_rms_norm(x, m._linear(y.transpose(1, 2).reshape(B, 1, c.n_embd), L["c_proj"]),
                                        L["ln_2"], c.norm_eps)
                if 0 < B <= m.decode_linear_rows:
                    mlp = m._mlp(L, h)
                else:
                    mlp = F.linear(ops.silu_mul(F.linear(h, L["c_fc2"]), F.linear(h, L["c_fc"])), L["mlp_proj"])
                next_norm = m.layers[i + 1]["ln_1"] if i + 1 < len(m.layers) else m.ln_f
                x, h = ops.add_rms_norm(x, mlp, next_norm, c.norm_eps)
            logits = m._linear(h[:, -1], m.wte)
        if hasattr(ops, "greedy_step"):
            # argmax and generate()'s bookkeeping (model.py:371-378) in two launches
            ops.greedy_step(logits, self.tokens, self.text_mask, self.tok, self.pos, self.kv_len, self.eos, self.stop)
            return
        nxt = ops.argmax(logits)   # first maximum of the bf16 logits = argmax of their float copy
        # generate() bookkeeping (model.py:373-378) at position pos + 1, all on the device
        cur = (self.pos + 1).long().clamp_(max=self.total_len - 1)
        keep = self.text_mask.index_select(1, cur).squeeze(1)
        nxt = torch.where(keep, self.tokens.index_select(1, cur).squeeze(1), nxt)
        self.tokens.index_copy_(1, cur, nxt.unsqueeze(1))
        self.eos |= ~keep & torch.isin(nxt, self.stop)
        self.tok.copy_(nxt.unsqueeze(1))
        self.pos += 1
        self.kv_len += 1

    MAX_PREFILL_GRAPHS = 4

    def prefill(self, m: "LlamaDecoder", T: int):
        """Logits of the prompt's first T positions (model.py:365 with start_pos 0) for the tokens in
        self.tokens.  The eager pass costs ~260 launches from Python (3.3 ms at batch 1, against 0.64 ms
        for a decode step), so it is recorded too, once per prompt length.  A recorded pass is used only
        after it has reproduced the eager logits bit for bit on two replays with eager work in between
        (library GEMMs may record nodes that misbehave on later replays); otherwise the eager pass stays."""
        import gc

        entry = self.prefill_graphs.get(T)
        if entry is None:
            # a recording keeps its activations' memory for as long as it lives: only the last few prompt
            # lengths stay recorded
            while len(self.prefill_graphs) >= self.MAX_PREFILL_GRAPHS:
                self.prefill_graphs.pop(next(iter(self.prefill_graphs)))
            dev = m.device
            ref = m.forward(self.tokens[:, :T], start_pos=0).clone()   # eager: also the warm-up for the capture
            torch.cuda.synchronize(dev)
            graph, out = None, None
            gc.collect()
            gc_was_enabled = gc.isenabled()
            gc.disable()
            ok = True
            try:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    out = m.forward(self.tokens[:, :T], start_pos=0)
            except RuntimeError:
                # an operator of the prompt pass refused to be recorded (the context manager has ended the
                # capture): this length stays eager
                ok = False
                torch.cuda.synchronize(dev)
            finally:
                if gc_was_enabled:
                    gc.enable()
            for _ in range(2 if ok else 0):
                graph.replay()
                torch.cuda.synchronize(dev)
                ok = ok and bool(torch.equal(out, ref))
                again = m.forward(self.tokens[:, :T], start_pos=0)      # eager work between the replays
                ok = ok and bool(torch.equal(again, ref))
            entry = (graph, out) if ok else (None, None)
            self.prefill_graphs[T] = entry
        if entry[0] is None:
            return m.forward(self.tokens[:, :T], start_pos=0)
        entry[0].replay()
        return entry[1]

    def capture(self, m: "LlamaDecoder"):
        import gc

        state = (self.tokens, self.tok, self.pos, self.kv_len, self.eos)
        saved = [t.clone() for t in state]
        side = torch.cuda.Stream(device=m.device)
        side.wait_stream(torch.cuda.current_stream(m.device))
        with torch.cuda.stream(side):
            self.step(m)   # warm-up outside capture: workspaces, hipBLASLt handles, allocator
        torch.cuda.current_stream(m.device).wait_stream(side)
        torch.cuda.synchronize(m.device)
        for t, s in zip(state, saved):
            t.copy_(s)
        # No garbage collection while the stream is capturing: a collected CUDAGraph or cached
        # block would be freed with calls that are illegal during capture.
        gc.collect()
        gc_was_enabled = gc.isenabled()
        gc.disable()
        try:
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.step(m)
        finally:
            if gc_was_enabled:
                gc.enable()
        for t, s in zip(state, saved):
            t.copy_(s)   # capture does not execute, but keep the state explicit
        torch.cuda.synchronize(m.device)


def random_prompts(batch, length, vocab_size, seed, exclude=(128004, 128001)):
    """Uniform random token ids from a seeded generator, avoiding the pad and stop ids
    (benchmark_model.py:17-43 draws from the tokenizer's vocabulary and avoids EOS)."""
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, vocab_size, (batch, length), generator=g)
    for e in exclude:
        ids = torch.where(ids == e, (ids + 1) % vocab_size, ids)
    return ids.tolist()


def timed_generate(model, batch, input_len, gen_len, seed=42, sync=None, graphed=False):
    """tokens/s = gen_len * batch / wall time of generate(), prefill included (benchmark_model.py:76-82)."""
    prompts = random_prompts(batch, input_len, model.config.vocab_size, seed)
    if sync:
        sync()
    t0 = time.perf_counter()
    if graphed:
        out = model.generate_graphed(prompts, max_gen_len=gen_len, ignore_eos=True)
    else:
        out = model.generate(prompts, max_gen_len=gen_len, temperature=0.0, ignore_eos=True)
    if sync:
        sync()
    dt = time.perf_counter() - t0
    return gen_len * batch / dt, dt, out


def e2e_summary(torch_mod, dev, batches=(1, 64), input_len=128, gen_len=128, repeats=2, cpu_ops=None):
    """The end-to-end configuration in short form, for the default benchmark line: per batch size the
    graph-replayed greedy decode (best of `repeats` after one warm-up generation that also records the
    graph) in tokens/s and microseconds per generated token, the eager loop beside it, and how many of the
    generated tokens the two loops agree on; with `cpu_ops` (an operator table working on CPU tensors) a
    shortened batch-1 generation of the same model on the host cores."""
    import os

    from custom_kernels import custom_kernels_extension as cke

    sync = torch_mod.cuda.synchronize
    cfg = LlamaConfig(max_model_len=input_len + gen_len, max_gen_batch_size=max(batches))
    model = LlamaDecoder(cfg, cke, dev)
    out = {}
    for batch in batches:
        timed_generate(model, batch, input_len, 2, seed=1)                       # eager warm-up
        eager_tps, _, eager_toks = timed_generate(model, batch, input_len, gen_len, sync=sync)
        timed_generate(model, batch, input_len, gen_len, seed=1, graphed=True)   # records the graph
        best, toks = 0.0, None
        for _ in range(repeats):
            tps, _, t = timed_generate(model, batch, input_len, gen_len, sync=sync, graphed=True)
            if tps > best:
                best, toks = tps, t
        same = sum(a == b for ra, rb in zip(eager_toks, toks) for a, b in zip(ra, rb))
        out[f"bs{batch}"] = {"tok_per_s": round(best, 1), "us_per_generated_token_step": round(1e6 * batch / best, 1),
                             "eager_tok_per_s": round(eager_tps, 1),
                             "graphed_vs_eager_same_tokens": f"{same}/{batch * gen_len}",
                             "prefill_pass": model.prefill_pass_mode(),
                             "weight_stream_frac_of_hbm_peak": round(2471628800 * best / batch / 8e12, 4)}
    out["config"] = (f"Llama-3.2-1B architecture, random init, {input_len} prompt ids + {gen_len} greedy tokens, "
                     "prefill included, decode loop replayed from a HIP graph")
    if cpu_ops is not None:
        cpu_model = LlamaDecoder(LlamaConfig(max_model_len=input_len + gen_len, max_gen_batch_size=1), cpu_ops, "cpu",
                                 weights_from=model)
        short = 8
        tps, dt, _ = timed_generate(cpu_model, 1, input_len, short)
        out["cpu_baseline"] = {"value": round(tps, 2), "unit": "tokens/s", "cores": torch_mod.get_num_threads(),
                               "kind": "port", "host_cpus": os.cpu_count(),
                               "sample": f"same model and prompts on the CPU with torch ops, batch 1, {input_len} prompt "
                                         f"ids + {short} greedy tokens in {dt:.1f} s (shortened generation)"}
        del cpu_model
    del model
    torch_mod.cuda.empty_cache()
    return out


def bench_e2e(args, torch_mod, dev, cpu_ops=None):
    """bench.py --workload e2e: the end-to-end configuration (16 layers, hidden 2048, 32/8 heads, head_dim 64,
    FFN 8192, vocab 128256 tied, N(0, 0.02) weights, 128 random prompt ids + 128 greedy tokens) at
    batch 1 and 64, every RMSNorm / rotary / decode-attention call going through the HIP operators.
    `cpu_ops` (an object with rms_norm, rot_embed and flash_attention_decode working on CPU tensors) is the
    caller's operator table for the timed CPU baseline; without one no baseline is reported."""
    import os

    from custom_kernels import custom_kernels_extension as cke

    input_len, gen_len = 128, 128
    results = {}
    for batch in (1, 64):
        cfg = LlamaConfig(max_model_len=input_len + gen_len, max_gen_batch_size=batch)
        model = LlamaDecoder(cfg, cke, dev)
        rec = {}
        # stock F.linear (hipBLASLt) in the decode step first, for the comparison ...
        model.set_decode_linear_rows(0)
        timed_generate(model, batch, input_len, gen_len, seed=1, graphed=True)
        best = max(timed_generate(model, batch, input_len, gen_len, sync=torch_mod.cuda.synchronize, graphed=True)[0]
                   for _ in range(3))
        rec["graphed_torch_linear"] = {"tok_per_s": round(best, 1)}
        # ... then the library's weight-streaming linear kernels where they apply (up to 16 rows)
        model.set_decode_linear_rows(16)
        rec["decode_linear"] = ("l3_linear_decode (fused)" if 0 < batch <= model.decode_linear_rows else
                                "l3_linear_splitk for c_attn / c_proj / mlp c_proj, F.linear for gate|up and lm_head"
                                if model._splitk(batch) else "torch F.linear")
        for mode in ("eager", "graphed"):
            graphed = mode == "graphed"
            # warm-up generate, as llama3_inference.py:31-36 does (for the graphed loop it also records the graph)
            timed_generate(model, batch, input_len, gen_len if graphed else 2, seed=1, graphed=graphed)
            best, toks = 0.0, None
            for _ in range(3):
                tps, dt, out = timed_generate(model, batch, input_len, gen_len, sync=torch_mod.cuda.synchronize,
                                              graphed=graphed)
                if tps > best:
                    best, toks = tps, out
            rec[mode] = {"tok_per_s": round(best, 1), "seconds": round(gen_len * batch / best, 4)}
            rec[mode + "_tokens"] = toks
        same = sum(a == b for ra, rb in zip(rec.pop("eager_tokens"), rec.pop("graphed_tokens")) for a, b in zip(ra, rb))
        rec["graphed_vs_eager_same_tokens"] = f"{same}/{batch * gen_len}"
        rec["prefill"] = model.prefill_backend
        rec["prefill_pass"] = model.prefill_pass_mode()
        results[batch] = rec
        del model
        torch_mod.cuda.empty_cache()

    cpu = None
    if cpu_ops is not None:
        cfg = LlamaConfig(max_model_len=input_len + gen_len, max_gen_batch_size=1)
        cpu_model = LlamaDecoder(cfg, cpu_ops, "cpu")
        short = 16
        tps, dt, _ = timed_generate(cpu_model, 1, input_len, short)
        cpu = {"value": round(tps, 2), "unit": "tokens/s", "cores": torch_mod.get_num_threads(), "kind": "port",
               "host_cpus": os.cpu_count(),
               "sample": f"same architecture and prompts on the CPU with torch ops, batch 1, 128 prompt ids + "
                         f"{short} greedy tokens in {dt:.1f} s (shortened generation)"}

    v = results[1]["graphed"]["tok_per_s"]
    return {
        "metric": "e2e_greedy_decode_tokens_per_s_bs1", "value": v, "unit": "tokens/s", "steps": args.steps,
        "ms_per_step": round(1e3 / v, 4), "dtype": "bf16",
        "config": {"workload": "Llama-3.2-1B architecture, random init, 128 prompt ids + 128 greedy tokens, batch 1 "
                               "(batch 64 alongside); a step is one generated token; decode loop replayed from a "
                               "HIP graph (the eager loop is reported next to it)", "seed": 42},
        "roofline": {"bound": "hbm", "achieved": round(2471628800 * v / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                     "frac": round(2471628800 * v / 1e9 / 8000.0, 4), "traffic": None,
                     "note": "bf16 weight bytes streamed per generated token x tokens/s; launch-bound at batch 1"},
        "cpu_baseline": cpu,
        "e2e": {"bs1": results[1], "bs64": results[64]},
    }
