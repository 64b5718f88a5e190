"""Text generation loops -- API of ``llm_quest/generate.py`` for the paths on SURVEY.md section 8 row f4: ``generate_loop``
(full re-forward per token), ``generate_loop_kv_cache`` (prefill + one-token decode steps through ``KVCache``) and ``sampling``.

Greedy sampling (``temp == 0``, the default) is a HIP kernel (first index of the row maximum).  Stochastic sampling (temperature /
top-k / top-p / min-p) is control logic on a (batch, vocab) tensor per generated token, outside the measured path: it is restated
here with torch device ops so the loops are complete, and says so.
"""

import torch

from . import ops_decode
from .utils import KVCache


def _top_k(probs, k):
    top, idx = torch.topk(probs, k)
    return torch.zeros_like(probs).scatter_(-1, idx, top)


def _top_p(probs, p, top_k=None):
    if top_k:
        kth = torch.topk(probs, top_k)[0][..., -1].unsqueeze(-1)
        probs = probs.masked_fill(probs < kth, 0.0)
    sp, idx = torch.sort(probs, dim=-1, descending=True)
    mask = torch.cumsum(sp, dim=-1) > p
    mask[..., 1:] = mask[..., :-1].clone()
    mask[..., 0] = False
    return torch.zeros_like(probs).scatter_(-1, idx, sp.masked_fill(mask, 0.0))


def _min_p(probs, min_p, min_tokens_to_keep=1):
    remove = probs < min_p * torch.amax(probs, dim=-1, keepdim=True)
    keep_idx = torch.topk(probs, min_tokens_to_keep)[1]
    remove.scatter_(-1, keep_idx, False)
    return probs.masked_fill(remove, 0.0)


def sampling(logits, top_k=None, top_p=None, min_p=None, temp=0.0):
    """logits (b, v) -> next token ids (b, 1) (reference: generate.py:472-514)."""
    assert top_p is None or min_p is None, "Cannot use top_p and min_p together"
    if temp == 0.0:
        return ops_decode.argmax_rows(logits if logits.stride(-1) == 1 else logits.contiguous()).unsqueeze(-1)
    probs = torch.softmax(logits.float() / temp, dim=-1)
    if min_p:
        probs = _min_p(probs, min_p, 1 if top_k is None else top_k)
    elif top_p:
        probs = _top_p(probs, top_p, top_k)
    elif top_k:
        probs = _top_k(probs, top_k)
    probs = probs / probs.sum(dim=-1, keepdim=True)
    return torch.multinomial(probs, num_samples=1)


def generate_loop(input_tensor, model, max_gen, context_length, top_k=None, top_p=None, min_p=None, temp=0.0, eos_ids=None, device=torch.device("cuda")):
    """Re-runs the model on the growing sequence for every token (reference: generate.py:29-94)."""
    input_tensor = input_tensor.to(device)
    eos = None
    if eos_ids is not None:
        eos = torch.tensor(eos_ids if isinstance(eos_ids, list) else [eos_ids], device=device, dtype=torch.long)
    for _ in range(max_gen):
        with torch.inference_mode():
            logits = model(input_tensor[:, -context_length:])[:, -1, :]
        next_token = sampling(logits, top_k, top_p, min_p, temp)
        if eos is not None and torch.isin(next_token, eos).any():
            break
        input_tensor = torch.cat((input_tensor, next_token), dim=-1)
    return input_tensor


def generate_loop_kv_cache(input_tensor, model, max_gen, context_length, top_k=None, top_p=None, min_p=None, temp=0.0, eos_ids=None,
                           device=torch.device("cuda"), use_graph=True):
    """Prefill once, then one-token decode steps through the KV cache (reference: generate.py:97-151).  Greedy decoding
    (``temp == 0``) replays one captured hipGraph per token (``use_graph``); sampling runs the steps eagerly."""
    if use_graph and temp == 0.0 and max_gen > 0 and hasattr(model, "trf_blocks") and input_tensor.shape[-1] + max_gen <= context_length:
        return _generate_greedy_graph(input_tensor, model, max_gen, context_length, eos_ids, device)
    token_ids = []
    kv_cache = KVCache(num_layers=len(model.trf_blocks), prompt_len=input_tensor.shape[-1], context_len=context_length)
    input_tensor = input_tensor.to(device)
    eos = None
    if eos_ids is not None:
        eos = torch.tensor(eos_ids if isinstance(eos_ids, list) else [eos_ids], device=device, dtype=torch.long)
    trunc_input = input_tensor[:, -context_length:]
    next_position_id = torch.tensor([[trunc_input.shape[-1]]], dtype=torch.long, device=device)
    with torch.inference_mode():
        logits = model(trunc_input, kv_cache=kv_cache)[:, -1, :]
        for _ in range(max_gen):
            next_token = sampling(logits, top_k, top_p, min_p, temp)
            if eos is not None and torch.isin(next_token, eos).any():
                break
            token_ids.append(next_token)
            logits = model(next_token, kv_cache=kv_cache, position_ids=next_position_id).squeeze(1)
            next_position_id += 1
    return torch.cat([input_tensor] + token_ids, dim=-1)


def _generate_greedy_graph(input_tensor, model, max_gen, context_length, eos_ids, device):
    token_ids = []
    kv_cache = KVCache(num_layers=len(model.trf_blocks), prompt_len=input_tensor.shape[-1], context_len=context_length)
    input_tensor = input_tensor.to(device)
    eos = None
    if eos_ids is not None:
        eos = torch.tensor(eos_ids if isinstance(eos_ids, list) else [eos_ids], device=device, dtype=torch.long)
    with torch.inference_mode():
        logits = model(input_tensor[:, -context_length:], kv_cache=kv_cache)[:, -1, :]
        next_token = sampling(logits)
        dec = None
        try:
            for _ in range(max_gen):
                if eos is not None and torch.isin(next_token, eos).any():
                    break
                token_ids.append(next_token)
                if len(token_ids) == max_gen:
                    break
                if dec is None:
                    dec = ops_decode.GraphDecoder(model, kv_cache, next_token, max_gen)
                next_token = dec.step()
        finally:
            if dec is not None:
                dec.close()
    return torch.cat([input_tensor] + token_ids, dim=-1)


def _batched_kv_loop(input_tensor, model, max_gen, context_length, top_k, top_p, min_p, temp, eos_ids, pad_id, device, attention_mask,
                     first_position_ids, next_pos_ids, pick_first_logits):
    """Shared body of the two padded, batched KV-cache loops: prefill, then one token per unfinished sequence; finished sequences keep
    receiving ``pad_id`` and are masked out of later attention (reference: generate.py:252-365, 368-469)."""
    input_tensor = input_tensor.to(device)
    attention_mask = attention_mask.bool().to(device)
    eos = torch.tensor(eos_ids if isinstance(eos_ids, list) else [eos_ids], device=device, dtype=torch.long)
    pad = torch.tensor(pad_id, device=device, dtype=torch.long)
    finished = torch.zeros(input_tensor.shape[0], dtype=torch.bool, device=device)
    kv_cache = KVCache(num_layers=len(model.trf_blocks), prompt_len=input_tensor.shape[-1], context_len=context_length)
    generated = []
    with torch.inference_mode():
        logits = pick_first_logits(model(input_tensor, attn_mask=attention_mask, kv_cache=kv_cache, position_ids=first_position_ids))
        for i in range(max_gen):
            next_token = torch.where(finished.unsqueeze(-1), pad, sampling(logits, top_k, top_p, min_p, temp))
            generated.append(next_token)
            finished |= torch.isin(next_token.squeeze(1), eos)
            attention_mask = torch.cat([attention_mask, (~finished).unsqueeze(-1)], dim=-1)
            if finished.all():
                break
            if i < max_gen - 1:
                logits = model(next_token, attn_mask=attention_mask, kv_cache=kv_cache, position_ids=next_pos_ids).squeeze(1)
            next_pos_ids = next_pos_ids + 1
    return torch.cat([input_tensor] + generated, dim=1)


def generate_batched_loop_kv_cache(input_tensor, model, max_gen, context_length, top_k=None, top_p=None, min_p=None, temp=0.0, eos_ids=50256,
                                   pad_id=50256, device=torch.device("cuda"), last_real=None, *, attention_mask):
    """RIGHT-padded prompts: the first logits come from each sequence's last real token, rotary positions continue from its real
    length (reference: generate.py:252-365)."""
    attention_mask = attention_mask.bool().to(device)
    if last_real is not None:
        last_real = last_real.to(device)
        next_pos = last_real.unsqueeze(-1) + 1
    else:
        next_pos = attention_mask.sum(dim=-1, keepdim=True)
        last_real = next_pos.squeeze(-1) - 1
    rows = torch.arange(input_tensor.shape[0], device=device)
    return _batched_kv_loop(input_tensor, model, max_gen, context_length, top_k, top_p, min_p, temp, eos_ids, pad_id, device, attention_mask,
                            None, next_pos, lambda lg: lg[rows, last_real, :])


def generate_batched_loop_kv_cache_left_pad(input_tensor, model, max_gen, context_length, top_k=None, top_p=None, min_p=None, temp=0.0,
                                            eos_ids=50256, pad_id=50256, device=torch.device("cuda"), *, attention_mask):
    """LEFT-padded prompts: positions count real tokens only (pads sit at position 0), every sequence ends in the last column
    (reference: generate.py:368-469)."""
    attention_mask = attention_mask.bool().to(device)
    position_ids = (attention_mask.cumsum(dim=-1) - 1).masked_fill(~attention_mask, 0)
    next_pos = attention_mask.sum(dim=-1, keepdim=True)
    return _batched_kv_loop(input_tensor, model, max_gen, context_length, top_k, top_p, min_p, temp, eos_ids, pad_id, device, attention_mask,
                            position_ids, next_pos, lambda lg: lg[:, -1, :])


# ----------------------------------------------------------------------------------------------- ragged batches (slot cache, no padding)
class RaggedBatch:
    """Scheduler of the serving models of ``registry`` (``model.step`` + ``utils.SlotStateCache``): sequences of different lengths run as ONE packed
    batch without padding.  A step brings, for every sequence in it, its next tokens -- a whole prompt for a sequence that starts, one token (or more) for
    one that goes on -- and returns fp32 logits of the rows asked for.  Sequences are named by the caller; ``finish`` gives a sequence's slot back, and
    the next sequence to start takes it.  A row's logits do not depend on which other sequences share the step."""

    def __init__(self, model, max_tokens=0, slots=4, device=None):
        self.model = model
        self.device = device or next(model.parameters()).device
        # max_tokens is a hint for the rows a slot starts with (rows grow on demand, so a generous hint must not reserve slots x hint rows up front)
        self.cache = model.new_cache(self.device, max_tokens=min(int(max_tokens), 8192), slots=slots)

    def step(self, entries, want=None, return_layers=False):
        """entries: [(seq_id, [token, ...])] in batch order.  want: per entry the positions among ITS new tokens whose logits are asked for (default:
        the last one).  Returns fp32 [rows asked for, vocab] in the order of the entries and of ``want`` (None if nothing is asked for)."""
        from .common.mixers import SeqStep

        if not entries:
            return None
        cache, vocab = self.cache, self.model.vocab_size
        slotted = []
        import numpy as np

        for seq_id, toks in entries:
            toks = np.asarray(toks, dtype=np.int64).reshape(-1)
            if toks.size and (int(toks.min()) < 0 or int(toks.max()) >= vocab):
                raise ValueError(f"sequence {seq_id!r}: token id outside [0, {vocab})")
            slot = cache.slot(seq_id) if seq_id in cache else cache.open(seq_id)
            slotted.append((slot, toks))
        st = SeqStep(cache, slotted, self.device, self.model.act_dtype)
        rows = []
        for i, (_, toks) in enumerate(slotted):
            w = [len(toks) - 1] if want is None else want[i]
            for p in w:
                if not 0 <= p < len(toks):
                    raise ValueError("a wanted position lies outside the entry's tokens")
                rows.append(st.host_seq_off[i] + p)
        # the whole stack runs even when no logits are asked for: the step still has to leave its rows and state behind
        want_rows = torch.tensor(rows if rows else [0], dtype=torch.long).to(self.device)
        out = self.model.step(st, want_rows, return_layers=return_layers)
        for slot, toks in slotted:
            cache.advance(slot, toks)
        if return_layers:
            return (out[0] if rows else None), out[1]
        return out if rows else None

    def finish(self, seq_id):
        if seq_id in self.cache:
            self.cache.close(seq_id)


def generate_ragged(model, prompts, max_gen, top_k=None, top_p=None, min_p=None, temp=0.0, eos_ids=None, max_tokens=0):
    """Generation for a list of prompts of different lengths (lists of token ids) through ``RaggedBatch``: all prompts start together in one packed
    step, then every unfinished sequence goes on by one sampled token per step; a sequence that produced an eos id (or ``max_gen`` tokens) leaves the
    batch and frees its slot.  Returns the generated ids per prompt (eos not included)."""
    eos = set(eos_ids if isinstance(eos_ids, (list, tuple, set)) else ([] if eos_ids is None else [eos_ids]))
    batch = RaggedBatch(model, max_tokens=max_tokens, slots=max(1, len(prompts)))
    out = [[] for _ in prompts]
    live = list(range(len(prompts)))
    entries = [(i, list(prompts[i])) for i in live]
    for _ in range(max_gen):
        if not entries:
            break
        logits = batch.step(entries)
        nxt = sampling(logits, top_k, top_p, min_p, temp).view(-1).tolist()
        entries, still = [], []
        for i, t in zip(live, nxt):
            if t in eos:
                batch.finish(i)
                continue
            out[i].append(int(t))
            if len(out[i]) >= max_gen:
                batch.finish(i)
                continue
            entries.append((i, [int(t)]))
            still.append(i)
        live = still
    return out


def main(argv=None):
    """``python -m llm_quest_amd.generate --model DIR --prompt 5,17,3 --prompt 9,2 --max-gen 16``: greedy or sampled continuation of token-id prompts
    with a serving model chosen by the folder's config.json."""
    import argparse
    import json

    from . import registry

    ap = argparse.ArgumentParser(description="generate token ids with a serving model (ragged batch, slot cache)")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=sorted(registry.DTYPES))
    ap.add_argument("--prompt", action="append", required=True, help="comma-separated token ids; repeat for a batch")
    ap.add_argument("--max-gen", type=int, default=16)
    ap.add_argument("--temp", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=None)
    ap.add_argument("--top-p", type=float, default=None)
    ap.add_argument("--eos", type=int, action="append", default=None)
    a = ap.parse_args(argv)
    model = registry.load_model(a.model, a.dtype, "cuda")
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt]
    print(json.dumps(generate_ragged(model, prompts, a.max_gen, top_k=a.top_k, top_p=a.top_p, temp=a.temp, eos_ids=a.eos)))


if __name__ == "__main__":
    main()
