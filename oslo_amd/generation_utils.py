"""``model.generate``: greedy and beam-search decoding over a key/value cache,
with the repeated n-gram ban either on the host (the HuggingFace processor) or
on the device (``FusedNoRepeatNGramLogitsProcessor``).

The reference's generation code is a fork of HuggingFace's GenerationMixin
(oslo/generation_utils.py) whose one addition on this path is the switch
``fused_no_repeat_ngram_blocking`` (:423-434, :753-757). This file is not that
fork: it restates the two decoding modes the reference's kernel-fusion test
uses (tests/gpt2/gpt2_test_kernel_fusion.py:26-33: ``max_length``,
``min_length``, ``num_beams``, ``no_repeat_ngram_size``) with the same
argument names and the same beam-search rule (oslo/generation_utils.py:
1913-1990 and HuggingFace's BeamSearchScorer), for prompts of equal length
without padding. Sampling, beam groups, constraints and the other logits
processors are not provided.

While no sequence can end (no ``eos_token_id``, or the length is still below
``min_length``) a step does not synchronise with the host: the beam
bookkeeping stays on the device.

A decoding step of a small model is a few hundred launches of a few
microseconds each, and the host cannot issue them as fast as the device
finishes them. ``generate(..., graph=True)`` therefore keeps the key/value
cache in preallocated buffers of ``max_length`` slots (``StaticKV``), so that
every step has the same shapes, captures one step (beam reordering of the
cache, the key masks, the model's forward, the position increment) as a HIP
graph and replays it once per token. ``static_cache=True`` alone runs the same
steps without a graph (on any device).
"""

import torch

from .fused_kernels_utils import FusedNoRepeatNGramLogitsProcessor


class DynamicDecoder(object):
    """Steps over a key/value cache that grows by concatenation."""

    def __init__(self, model, use_cache):
        self.model, self.use_cache, self.past = model, use_cache, None

    def step(self, ids, beam_idx=None):
        past = self.past
        if past is not None and beam_idx is not None:
            past = tuple(tuple(t.index_select(0, beam_idx) for t in layer) for layer in past)
        feed = ids[:, -1:] if past is not None else ids
        out = self.model(feed, past_key_values=past, use_cache=self.use_cache)
        self.past = out["past_key_values"]
        return out["logits"][:, -1, :]


def _model_fingerprint(model):
    """What a captured step depends on besides its inputs: the classes of the
    modules (``fuse()`` changes them), the storage of every parameter and
    buffer (``.half()`` or loading weights replaces it) and the mode."""
    return (model.training,
            tuple(id(type(m)) for m in model.modules()),
            tuple(t.data_ptr() for t in model.parameters()),
            tuple(t.data_ptr() for t in model.buffers()))


class StaticDecoder(object):
    """Steps over static caches; optionally each step is one graph replay. The
    first ``step`` takes the whole prompt (an ordinary forward whose keys and
    values fill the caches), every later one the sequences grown by one token.
    ``restart()`` makes the next ``step`` a first one again: the buffers and
    the captured graphs are kept as long as the shapes stay the same."""

    def __init__(self, model, capacity, graph):
        # whole 64-key vectors: the key-mask softmax then takes its vector path
        self.model, self.capacity, self.graph = model, -(-int(capacity) // 64) * 64, graph
        self.caches = None
        self._captured = {}  # reorder flag -> (graph, logits)
        self._started = False

    def restart(self):
        self._started = False

    def _prefill(self, ids):
        from .modeling_utils import DecodeState, StaticKV

        out = self.model(ids, use_cache=True)
        presents = out["past_key_values"]
        k0 = presents[0][0]
        shape = (len(presents), 2, k0.size(0), k0.size(1), self.capacity, k0.size(3))
        if self.caches is None or tuple(self.store.shape) != shape or self.store.dtype != k0.dtype \
                or self.store.device != k0.device:
            self.state = DecodeState(self.capacity, ids.device, k0.dtype)
            self.store, self.caches = StaticKV.allocate(self.state, len(presents), k0.size(0), k0.size(1), k0.size(3),
                                                        k0.dtype, k0.device)
            self.token = ids[:, -1:].clone()
            self.beam_idx = torch.arange(ids.size(0), device=ids.device)
            self._captured = {}
        # slots past the prompt may hold an earlier sequence: they are hidden
        # until a step writes them
        for cache, (key, value) in zip(self.caches, presents):
            cache.pending = None
            cache.fill(key, value)
        self.state.pos.fill_(ids.size(1))
        self._started = True
        return out["logits"][:, -1, :]

    def _run(self, reorder):
        if reorder:  # every layer's keys and values follow their beams
            self.store.copy_(self.store.index_select(2, self.beam_idx))
        self.state.begin_step()
        logits = self.model(self.token, past_key_values=self.caches, use_cache=True)["logits"][:, -1, :]
        self.state.pos.add_(1)
        return logits

    def _capture(self, reorder):
        device = self.token.device
        pos = self.state.pos.clone()
        beam_idx = self.beam_idx.clone()
        # warm-up on a side stream: lazy initialisation must not happen inside
        # the capture. The warm-up steps really run: they write the slot of the
        # step, which the real step writes again, and advance the position,
        # which is put back; they reorder the caches by the identity, because
        # the step's own reordering must be applied once, by the replay.
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side):
            self.beam_idx.copy_(torch.arange(beam_idx.numel(), device=device))
            for _ in range(2):
                self._run(reorder)
                self.state.pos.copy_(pos)
            self.beam_idx.copy_(beam_idx)
        torch.cuda.current_stream(device).wait_stream(side)
        torch.cuda.synchronize(device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self._run(reorder)
        self.state.pos.copy_(pos)  # nothing ran during capture; keep the host-side view simple
        return graph, logits

    def step(self, ids, beam_idx=None):
        if not self._started:
            return self._prefill(ids)
        if int(ids.size(1)) > self.capacity:
            raise RuntimeError("generate: the static cache is full")
        self.token.copy_(ids[:, -1:])
        if beam_idx is not None:
            self.beam_idx.copy_(beam_idx)
        reorder = beam_idx is not None
        if not self.graph:
            return self._run(reorder)
        if reorder not in self._captured:
            self._captured[reorder] = self._capture(reorder)
        graph, logits = self._captured[reorder]
        graph.replay()
        return logits


class _HostNoRepeatNGram(object):
    """The unfused ban: HuggingFace's NoRepeatNGramLogitsProcessor, which walks
    the token lists on the host (what the reference uses when the switch is
    off, oslo/generation_utils.py:433-434)."""

    def __init__(self, ngram_size):
        from transformers.generation.logits_process import NoRepeatNGramLogitsProcessor

        self.processor = NoRepeatNGramLogitsProcessor(ngram_size)

    def __call__(self, input_ids, scores):
        return self.processor(input_ids, scores)


class _BeamHypotheses(object):
    """Finished sequences of one batch entry: the ``num_beams`` best by
    sum of log-probabilities / length ** length_penalty."""

    def __init__(self, num_beams, length_penalty):
        self.num_beams = num_beams
        self.length_penalty = length_penalty
        self.beams = []  # (score, tokens)
        self.worst = 1e9

    def add(self, tokens, sum_logprobs):
        score = sum_logprobs / (tokens.shape[-1] ** self.length_penalty)
        if len(self.beams) < self.num_beams or score > self.worst:
            self.beams.append((score, tokens))
            if len(self.beams) > self.num_beams:
                self.beams.sort(key=lambda b: b[0])
                del self.beams[0]
            self.worst = min(b[0] for b in self.beams)

    def is_done(self, best_sum_logprobs, cur_len):
        # no running beam can still beat the worst kept one
        if len(self.beams) < self.num_beams:
            return False
        return self.worst >= best_sum_logprobs / cur_len ** self.length_penalty


class GenerationMixin(object):
    """``generate`` for the causal language models of this package (their
    forward returns a dict with ``logits`` and ``past_key_values``)."""

    @torch.no_grad()
    def generate(self, input_ids, max_length=20, min_length=0, num_beams=1, no_repeat_ngram_size=None,
                 fused_no_repeat_ngram_blocking=None, eos_token_id=None, pad_token_id=None,
                 length_penalty=1.0, use_cache=True, static_cache=None, graph=False):
        if input_ids.dim() != 2:
            raise ValueError("generate: input_ids must be [batch, length]")
        if input_ids.size(1) >= max_length:
            raise ValueError(f"generate: the prompt ({input_ids.size(1)} tokens) leaves no room below max_length={max_length}")
        if num_beams < 1:
            raise ValueError("generate: num_beams must be at least 1")
        if fused_no_repeat_ngram_blocking is None:
            fused_no_repeat_ngram_blocking = bool(getattr(self.config, "fused_no_repeat_ngram_blocking", False))
        if eos_token_id is not None and pad_token_id is None:
            pad_token_id = eos_token_id
        batch = input_ids.size(0)
        static_cache = graph if static_cache is None else static_cache
        if graph:
            if not static_cache or not use_cache:
                raise ValueError("generate: graph=True decodes over the static cache")
            if not input_ids.is_cuda:
                raise RuntimeError("generate: graph=True needs the model and input_ids on a ROCm device")
            if self.training:
                raise RuntimeError("generate: graph=True captures inference: call model.eval() first")
        if static_cache and not use_cache:
            raise ValueError("generate: static_cache=True contradicts use_cache=False")
        if static_cache:
            decoder = self._static_decoder(max_length, graph)
        else:
            decoder = DynamicDecoder(self, use_cache)

        ban = None
        if no_repeat_ngram_size is not None and no_repeat_ngram_size > 0:
            if fused_no_repeat_ngram_blocking:
                ban = FusedNoRepeatNGramLogitsProcessor(no_repeat_ngram_size, batch, num_beams)
            else:
                ban = _HostNoRepeatNGram(no_repeat_ngram_size)

        def scores_of(ids, logits):
            s = torch.log_softmax(logits.float(), dim=-1) if num_beams > 1 else logits.float()
            if eos_token_id is not None and ids.size(1) < min_length:
                s[:, eos_token_id] = float("-inf")
            if ban is not None:
                s = ban(ids, s)
            return s

        if num_beams == 1:
            return self._greedy_search(input_ids, max_length, scores_of, eos_token_id, pad_token_id, decoder)
        return self._beam_search(input_ids, max_length, min_length, num_beams, scores_of, eos_token_id,
                                 pad_token_id, length_penalty, decoder)

    def _static_decoder(self, max_length, graph):
        """The decoder of the previous call when nothing it captured has
        changed (the graph of a step is worth keeping: capturing it costs as
        much as some twenty steps), else a new one."""
        if not graph:
            return StaticDecoder(self, max_length, False)
        key = (-(-int(max_length) // 64) * 64, _model_fingerprint(self))
        kept = self.__dict__.get("_kept_decoder")
        if kept is None or kept[0] != key:
            kept = (key, StaticDecoder(self, max_length, True))
            self.__dict__["_kept_decoder"] = kept
        kept[1].restart()
        return kept[1]

    def release_decoder(self):
        """Drops the decoder ``generate(graph=True)`` keeps between calls (its
        key/value buffers and captured graphs), e.g. before the model is
        pickled or to give the memory back."""
        self.__dict__.pop("_kept_decoder", None)

    @staticmethod
    def _greedy_search(ids, max_length, scores_of, eos_token_id, pad_token_id, decoder):
        unfinished = None if eos_token_id is None else torch.ones(ids.size(0), dtype=torch.bool, device=ids.device)
        while ids.size(1) < max_length:
            nxt = scores_of(ids, decoder.step(ids)).argmax(dim=-1)
            if unfinished is not None:
                nxt = torch.where(unfinished, nxt, torch.full_like(nxt, pad_token_id))
                unfinished = unfinished & (nxt != eos_token_id)
            ids = torch.cat([ids, nxt[:, None]], dim=-1)
            if unfinished is not None and not bool(unfinished.any()):
                break
        return ids

    def _beam_search(self, input_ids, max_length, min_length, num_beams, scores_of, eos_token_id, pad_token_id,
                     length_penalty, decoder):
        batch, dev = input_ids.size(0), input_ids.device
        ids = input_ids.repeat_interleave(num_beams, dim=0)
        beam_scores = torch.zeros((batch, num_beams), dtype=torch.float32, device=dev)
        beam_scores[:, 1:] = -1e9  # all beams start equal: only the first one counts at step 0
        beam_scores = beam_scores.view(-1)
        row0 = (torch.arange(batch, device=dev) * num_beams)[:, None]
        hyps = [_BeamHypotheses(num_beams, length_penalty) for _ in range(batch)]
        done = [False] * batch
        beam_idx = None

        while ids.size(1) < max_length:
            logits = decoder.step(ids, beam_idx)
            cur_len = ids.size(1)
            s = scores_of(ids, logits) + beam_scores[:, None]
            vocab = s.size(-1)
            top_s, top_i = torch.topk(s.view(batch, num_beams * vocab), 2 * num_beams, dim=1)
            src = torch.div(top_i, vocab, rounding_mode="floor")
            tok = top_i % vocab

            if eos_token_id is None or cur_len < min_length:
                # no candidate ends a sequence: the best num_beams continue
                beam_scores = top_s[:, :num_beams].reshape(-1)
                nxt = tok[:, :num_beams].reshape(-1)
                beam_idx = (row0 + src[:, :num_beams]).reshape(-1)
            else:
                beam_scores, nxt, beam_idx = self._select_on_host(
                    ids, top_s, tok, src, hyps, done, num_beams, eos_token_id, pad_token_id)
            ids = torch.cat([ids.index_select(0, beam_idx), nxt[:, None]], dim=-1)
            if all(done):
                break

        # what is still running competes with what has finished
        final_scores = beam_scores.view(batch, num_beams).tolist()
        best = []
        for b in range(batch):
            if not done[b]:
                for j in range(num_beams):
                    hyps[b].add(ids[b * num_beams + j], final_scores[b][j])
            best.append(max(hyps[b].beams, key=lambda h: h[0])[1])
        # a hypothesis does not hold its closing token: it is written back after
        # it, and the rest of the row is padding
        longest = min(max(t.size(0) for t in best) + 1, max_length)
        if any(t.size(0) < longest for t in best) and pad_token_id is None:
            raise ValueError("generate: sequences of different lengths need a pad_token_id")
        out = ids.new_full((batch, longest), 0 if pad_token_id is None else pad_token_id)
        for b, t in enumerate(best):
            out[b, : t.size(0)] = t
            if t.size(0) < max_length and eos_token_id is not None:
                out[b, t.size(0)] = eos_token_id
        return out

    @staticmethod
    def _select_on_host(ids, top_s, tok, src, hyps, done, num_beams, eos_token_id, pad_token_id):
        """One step of beam bookkeeping when sequences may end: candidates are
        visited best first; one that ends with ``eos_token_id`` becomes a
        finished hypothesis if it ranks among the first ``num_beams``, the
        others fill the next beams."""
        batch = top_s.size(0)
        cur_len = ids.size(1)
        s_l, t_l, i_l = top_s.tolist(), tok.tolist(), src.tolist()
        new_scores, new_tokens, new_idx = [], [], []
        for b in range(batch):
            if done[b]:
                new_scores += [0.0] * num_beams
                new_tokens += [pad_token_id] * num_beams
                new_idx += [b * num_beams] * num_beams
                continue
            taken = 0
            for rank, (sc, t, j) in enumerate(zip(s_l[b], t_l[b], i_l[b])):
                row = b * num_beams + j
                if t == eos_token_id:
                    if rank < num_beams:
                        hyps[b].add(ids[row].clone(), sc)
                else:
                    new_scores.append(sc)
                    new_tokens.append(t)
                    new_idx.append(row)
                    taken += 1
                if taken == num_beams:
                    break
            if taken < num_beams:
                raise RuntimeError("generate: fewer than num_beams candidates continue a sequence")
            done[b] = hyps[b].is_done(max(s_l[b]), cur_len)
        dev = ids.device
        return (torch.tensor(new_scores, dtype=torch.float32, device=dev),
                torch.tensor(new_tokens, dtype=torch.long, device=dev),
                torch.tensor(new_idx, dtype=torch.long, device=dev))
