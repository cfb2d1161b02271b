"""Greedy decode loop with the decode step captured into a HIP graph.

The reference issues ~227 kernel launches per token from Python through pybind
(muillm/sampling/generation.py:244-408 drives muillm/modules/models/llama/model.py:699-801)
and only has a single-call C++ decoder stack under tensor parallelism
(csrc/modules/parallel_decoder_stack.cpp). Here one decode step -- embedding gather, all
decoder layers, final norm, lm_head, argmax, and the advance of the position counters -- is
recorded once on a side stream and replayed; everything the step needs to know about "where
are we" lives in device memory (input ids, position ids, cache slot, output slot), and the
attention kernel reads the sequence length from the cache slot, so the graph never changes
as the sequence grows. No memset nodes are recorded: one hand-written kernel picks the token,
stores it, applies the eos criterion and advances every counter (the reference's torch.argmax
+ muillm_add_tokens_check_finished, muillm/sampling/generation.py:330-404)."""
from typing import Optional

import torch

from ... import muillm_ext
from ..kvcache.cache_utils import MuiStaticCache, _next_pow2, create_static_cache


class MuiGraphDecoder:
    # decode steps per graph replay when nothing has to happen between steps on the host (no stop
    # check due, no logits wanted): consecutive replays of a one-step graph start ~9 us apart from
    # each other's end, kernels inside a graph abut
    STEPS_PER_REPLAY = 4

    def __init__(self, lm, use_graph: Optional[bool] = True, eos_token_ids=None, pad_token_id: int = 0,
                 do_sample: bool = False, temperature: float = 1.0, seed: int = 0,
                 top_k: Optional[int] = None, top_p: Optional[float] = None):
        """do_sample=True draws from softmax(logits / temperature) on the device (the reference's
        sync-free multinomial, muillm/sampling/multinomial.py:4-6) instead of taking the argmax;
        the draws are a function of (seed, batch row, step), so a run is reproducible.

        use_graph: True replays the captured decode step, False enqueues every step's kernels on the
        stream, None chooses when the first step is due: stream launches where the whole layer stack
        is one library call (the host then needs ~0.8 ms for a 2.6 ms step of the 8B shape, and the
        rate is the same as or a little above graph replay -- 383-386 against 380-382 tokens/s at
        batch 1 -- without graph replay's slower first ~70 launches in a fresh process: 2.69 against
        2.62 ms per step), graph replay where the layers run as separate module calls and the host
        would be the limit."""
        self.lm = lm
        self._requested_mode = use_graph  # None: chosen again at every decode() call
        self.use_graph = use_graph
        self.do_sample = do_sample
        self.temperature = float(temperature)
        self.seed = int(seed)
        # top-k / top-p filtering runs as torch ops (topk / sort) in front of the sampling kernel;
        # those library calls stay out of HIP graphs, so the loop is eager when they are on
        self.top_k = int(top_k) if top_k else None
        self.top_p = float(top_p) if top_p is not None and top_p < 1.0 else None
        if self.top_k or self.top_p:
            self.use_graph = self._requested_mode = False
        self.eos_token_ids = list(eos_token_ids) if eos_token_ids is not None else None
        self.pad_token_id = int(pad_token_id)
        self.graph = None
        self.graph_multi = None  # STEPS_PER_REPLAY steps in one graph, captured on first use
        self._graph_key = None  # what the captured graph has baked in (see _capture_key)
        self.cache: Optional[MuiStaticCache] = None
        self.owns_cache = False  # True when prefill() created self.cache itself
        self._window = 0  # sliding window kept in mask4d by every step (0: none)
        self._embed_table = None
        self.mask4d = None
        self._batch = None

    # -- static device state shared by every replay --
    def _alloc_state(self, batch: int, max_new_tokens: int, device):
        self.ids = torch.zeros((batch, 1), dtype=torch.int64, device=device)
        self.pos = torch.zeros((batch, 1), dtype=torch.int64, device=device)
        self.cpos = torch.zeros((1,), dtype=torch.int64, device=device)
        self.step = torch.zeros((batch,), dtype=torch.int64, device=device)
        self.unfinished = torch.ones((batch,), dtype=torch.int64, device=device)
        self.eos = (torch.tensor(self.eos_token_ids, dtype=torch.int64, device=device)
                    if self.eos_token_ids else None)
        self.out_tokens = torch.zeros((batch, max_new_tokens), dtype=torch.int64, device=device)
        # lets the token choice scan a long vocabulary on several workgroups; returns to zero every step
        self._greedy_ws = muillm_ext.greedy_workspace(batch, device)
        # greedy decoding: the token choice leaves the chosen token's embedding row here, and the
        # next step starts from it instead of launching a gather (token id -> row: two dependent
        # loads at the head of every step)
        table = getattr(getattr(getattr(self.lm, "model", None), "embed_tokens", None), "weight", None)
        self._embed_table = None
        if (not self.do_sample and table is not None and table.is_cuda and table.dim() == 2 and table.stride(1) == 1
                and table.dtype in (torch.float16, torch.bfloat16)):
            self._embed_table = table
            self.hidden = torch.zeros((batch, 1, table.shape[1]), dtype=table.dtype, device=device)
        self.logits = None
        self.mask4d = None  # static additive decode mask [B, 1, 1, capacity] when the prompts are padded
        self._stop_host = None  # pinned scalar for the sync-free stop check
        self._batch = batch
        self._max_new = max_new_tokens

    def _step(self):
        """One decode step on the static buffers (this is what gets captured)."""
        fold = self._embed_table is not None
        if self._window:
            # sliding window (the reference's mistral/model.py:590-602): the token in slot c sees the
            # keys after c - window; the window only moves forward, so the keys it leaves behind
            # stay hidden in the static mask
            self.mask4d.masked_fill_(self._key_index <= (self.cpos - self._window), torch.finfo(self.mask4d.dtype).min)
        out = self.lm(input_ids=None if fold else self.ids, inputs_embeds=self.hidden if fold else None,
                      position_ids=self.pos, cache_position=self.cpos,
                      past_key_values=self.cache, use_cache=True, attention_mask=self.mask4d,
                      all_ones_mask=self.mask4d is None, float_logits=False)
        logits = out.logits[:, -1, :]
        self._advance(logits)
        return logits

    def _advance(self, logits):
        """Token choice + stop check + token store + counters: one launch, all on the device."""
        if self.do_sample:
            logits = self._filter_logits(logits)
            muillm_ext.mui_sample_advance(logits, self.ids, self.step, self.out_tokens, temperature=self.temperature,
                                          seed=self.seed, position_ids=self.pos, cache_position=self.cpos,
                                          unfinished=self.unfinished, eos_token_ids=self.eos,
                                          pad_token_id=self.pad_token_id)
        else:
            muillm_ext.mui_greedy_advance(logits, self.ids, self.step, self.out_tokens, position_ids=self.pos,
                                          cache_position=self.cpos, unfinished=self.unfinished,
                                          eos_token_ids=self.eos, pad_token_id=self.pad_token_id,
                                          workspace=self._greedy_ws, embed_table=self._embed_table,
                                          embed_out=self.hidden if self._embed_table is not None else None)

    def _filter_logits(self, logits):
        """HuggingFace's TopKLogitsWarper / TopPLogitsWarper on the temperature-scaled distribution:
        everything outside the k largest logits, or outside the smallest set of tokens whose
        probability mass reaches top_p, becomes -inf (the sampling kernel never draws those)."""
        if not (self.top_k or self.top_p):
            return logits
        lg = logits.float()
        if self.top_k:
            k = min(self.top_k, lg.shape[-1])
            kth = torch.topk(lg, k, dim=-1).values[..., -1:]
            lg = lg.masked_fill(lg < kth, float("-inf"))
        if self.top_p:
            srt, idx = torch.sort(lg / self.temperature, dim=-1, descending=False)
            cum = torch.softmax(srt, dim=-1).cumsum(dim=-1)
            drop = cum <= (1.0 - self.top_p)
            drop[..., -1:] = False  # always keep the most likely token
            lg = lg.masked_fill(drop.scatter(-1, idx, drop), float("-inf"))
        return lg.to(logits.dtype)

    def _capture_key(self):
        """Everything a captured step holds by address or by value: the cache tensors (re-allocated
        when the cache grows, which also changes the head stride and the capacity the kernels
        clamp to), the batch size and whether a padding mask is part of the step."""
        c = self.cache
        # the weights a captured step reads (the embedding table of the folded gather included): a
        # model moved with .to() or quantised again after the first generate() must be captured anew
        weights = hash(tuple(t.data_ptr() for t in self.lm.parameters()) + tuple(t.data_ptr() for t in self.lm.buffers()))
        return (id(c), self._batch, c.max_cache_len, tuple(t.data_ptr() for t in c.key_cache),
                tuple(t.data_ptr() for t in c.value_cache),
                None if self.mask4d is None else self.mask4d.data_ptr(), self._window, weights,
                None if self._embed_table is None else self._embed_table.data_ptr())

    def _capture(self):
        self.cache.device_length_mode = True
        seen = self.cache._seen_tokens
        # warm up on a side stream (allocator, lazy module state), then restore the cache counters
        saved = [t.clone() for t in self._step_state()]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._restore(saved, seen)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self._graph_logits = self._step()  # where every replay leaves its logits
        self.logits = self._graph_logits
        self.graph_multi = None
        self._graph_key = self._capture_key()
        # capture does not execute: the device state is as restored; the host counter moved once
        self.cache._seen_tokens = seen
        if self.cache.cpp_module is not None:
            self.cache.cpp_module.seen_tokens = seen

    def _capture_multi(self):
        """STEPS_PER_REPLAY steps as one graph (the one-step graph has been captured and warmed up
        before). Capture does not execute; only the host-side token counter moves and is put back."""
        self.cache.device_length_mode = True  # (prefill switches it off) lengths are read on the device
        seen = self.cache._seen_tokens
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(self.STEPS_PER_REPLAY):
                self._multi_logits = self._step()  # the last step's
        self.graph_multi = g
        self.cache._seen_tokens = seen
        if self.cache.cpp_module is not None:
            self.cache.cpp_module.seen_tokens = seen

    def _step_state(self):
        """The device tensors a decode step changes (besides the cache slot it writes)."""
        state = [self.ids, self.pos, self.cpos, self.step, self.out_tokens, self.unfinished]
        if self._embed_table is not None:
            state.append(self.hidden)
        return state

    def _restore(self, saved, seen):
        for dst, src in zip(self._step_state(), saved):
            dst.copy_(src)
        self.cache._seen_tokens = seen
        if self.cache.cpp_module is not None:
            self.cache.cpp_module.seen_tokens = seen

    @torch.no_grad()
    def prefill(self, input_ids: torch.LongTensor, max_new_tokens: int, cache: Optional[MuiStaticCache] = None,
                attention_mask: Optional[torch.Tensor] = None):
        """attention_mask [B, prompt_len] of 0/1 marks LEFT padding (0 = pad): padded slots stay
        masked for the whole generation and every row counts its rotary positions from its own
        first real token, as HuggingFace's generate does."""
        lm = self.lm
        device = input_ids.device
        batch, prompt_len = input_ids.shape
        padded = attention_mask is not None and not bool(torch.all(attention_mask == 1))
        # a cache that already holds tokens continues after them (multi-turn): slots and rotary
        # positions are offset by what it has seen
        past = 0 if cache is None else cache.get_seq_length()
        if past and padded:
            raise ValueError("a left-padded prompt needs an empty cache (call cache.reset() first)")
        total = past + prompt_len + max_new_tokens
        window = getattr(lm.config, "sliding_window", None)
        windowed = bool(window) and total > int(window)  # decided for the whole generation: a captured step keeps its mask
        max_pos = lm.model.rotary_emb.max_seq_len_cached
        if total > max_pos:
            raise ValueError(f"cached tokens + prompt + max_new_tokens = {total} exceeds the {max_pos} rotary "
                             "positions of this model (max_position_embeddings)")
        self.owns_cache = cache is None or (cache is self.cache and self.owns_cache)
        if cache is None:
            cache = create_static_cache(lm.engine_config, lm.config, batch, total, device, lm.model.mdtype)
        else:
            if batch > cache.max_batch_size:
                raise ValueError(f"batch {batch} exceeds the cache's max_batch_size {cache.max_batch_size}")
            if cache.max_cache_len < total:
                cache.grow_cache(total, max(lm.config.max_position_embeddings, _next_pow2(total)))
        self.cache = cache
        cache.device_length_mode = False
        if padded:
            am = attention_mask.to(device=device, dtype=torch.int64)
            if bool((am[:, -1] == 0).any()):
                raise ValueError("padding must be on the left: the last prompt position of every row must be real")
            prompt_pos = (am.cumsum(-1) - 1).clamp_(min=0)
            out = lm(input_ids=input_ids, attention_mask=am, position_ids=prompt_pos, past_key_values=cache,
                     use_cache=True, all_ones_mask=False, num_logits_to_keep=1, float_logits=False)
        else:
            out = lm(input_ids=input_ids, past_key_values=cache, use_cache=True, all_ones_mask=True,
                     num_logits_to_keep=1, float_logits=False)
        if self._batch != batch or getattr(self, "_max_new", 0) < max_new_tokens:
            self._alloc_state(batch, max_new_tokens, device)
            self.graph = None
        if padded or windowed:
            mdtype = lm.model.mdtype
            if self.mask4d is None or self.mask4d.shape[-1] != cache.max_cache_len or self.mask4d.shape[0] != batch:
                self.mask4d = torch.zeros((batch, 1, 1, cache.max_cache_len), dtype=mdtype, device=device)
            self.mask4d.zero_()
            if padded:
                self.mask4d[:, 0, 0, :prompt_len].masked_fill_(am == 0, torch.finfo(mdtype).min)
            self._key_index = torch.arange(cache.max_cache_len, device=device)
        else:
            self.mask4d = None
        self._window = int(window) if windowed else 0
        # a captured step is only good for the buffers it was recorded on
        if self.graph is not None and self._graph_key != self._capture_key():
            self.graph = None
        # the first new token goes through the same kernel as all later ones: the counters start
        # one step back and the launch advances them to (prompt_len, prompt_len, 1)
        if padded:
            self.pos.copy_(am.sum(-1, keepdim=True) - 1)
        else:
            self.pos.fill_(past + prompt_len - 1)
        self.cpos.fill_(past + prompt_len - 1)
        self.step.zero_()
        # columns never reached (early stop) read as padding
        self.out_tokens.fill_(self.pad_token_id if self.eos is not None else 0)
        self.unfinished.fill_(1)
        self._advance(out.logits[:, -1, :])
        return out.logits[:, -1, :]

    @torch.no_grad()
    def decode(self, n_steps: int, collect_logits: bool = False, stop_check_every: int = 0):
        """Run up to n_steps decode steps from the current device state.

        stop_check_every > 0 (and an eos criterion): every that many steps the count of unfinished
        rows is copied to pinned host memory WITHOUT waiting for it; the loop ends once a copy that
        has already landed reads zero. The host therefore never blocks on the GPU (the reference
        gets the same effect with its Synchronizer, csrc/sync.cu:16-118, muillm/sampling/generation.py);
        the few steps issued past the end only write pad tokens."""
        logits_hist = []
        if self._requested_mode is None:
            # chosen per call: another batch size or a caller's cache may change what the layer stack takes
            model = getattr(self.lm, "model", None)
            stack = model._decode_stack(self.cache, self._batch, self.ids) if hasattr(model, "_decode_stack") else None
            self.use_graph = stack is None
        if self.use_graph and self.graph is None:
            self._capture()
        if not self.use_graph:
            self.cache.device_length_mode = False
        check = stop_check_every > 0 and self.eos is not None
        pending = None  # (event, pinned host tensor) of the last stop-check copy
        done = 0
        if self.use_graph and not check and not collect_logits and self.graph_multi is None:
            self._capture_multi()  # on the first such call, however short: a later long one finds it ready
        if self.use_graph and not check and not collect_logits and n_steps >= 2 * self.STEPS_PER_REPLAY:
            # nothing to do on the host between steps: several steps per replay
            for _ in range(n_steps // self.STEPS_PER_REPLAY):
                self.graph_multi.replay()
            self.logits = self._multi_logits
            done = n_steps - n_steps % self.STEPS_PER_REPLAY
        for i in range(done, n_steps):
            if check and pending is not None and pending[0].query():
                if int(pending[1].item()) == 0:
                    break
                pending = None
            if self.use_graph:
                self.graph.replay()
                lg = self._graph_logits
            else:
                lg = self._step()
            self.logits = lg  # logits of the last step taken
            done += 1
            if collect_logits:
                logits_hist.append(lg.clone())
            if check and pending is None and (i + 1) % stop_check_every == 0:
                if self._stop_host is None:
                    self._stop_host = torch.zeros((), dtype=torch.int64, pin_memory=True)
                self._stop_host.copy_(self.unfinished.sum(), non_blocking=True)
                ev = torch.cuda.Event()
                ev.record()
                pending = (ev, self._stop_host)
        if self.use_graph:
            self.cache._seen_tokens += done
            if self.cache.cpp_module is not None:
                self.cache.cpp_module.seen_tokens = self.cache._seen_tokens
        return logits_hist

    @torch.no_grad()
    def generate(self, input_ids: torch.LongTensor, max_new_tokens: int, cache: Optional[MuiStaticCache] = None,
                 return_logits: bool = False, attention_mask: Optional[torch.Tensor] = None,
                 stop_check_every: int = 0):
        first_logits = self.prefill(input_ids, max_new_tokens, cache, attention_mask=attention_mask)
        hist = self.decode(max_new_tokens - 1, collect_logits=return_logits, stop_check_every=stop_check_every)
        tokens = torch.cat([input_ids, self.out_tokens[:, :max_new_tokens]], dim=1)
        if return_logits:
            return tokens, torch.stack([first_logits] + hist, dim=1)
        return tokens
