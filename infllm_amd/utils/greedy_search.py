"""Greedy generation with chunked prefill (inf_llm/utils/greedy_search.py:3-105).

The call schedule is part of the behaviour, because every model call becomes one ``append`` of the
per-layer memory and so decides where its execution blocks fall: the prompt WITHOUT its last token is fed
in pieces of ``chunk_size``, then the last token alone, then one token per generated step; the per-layer
caches returned by the model are carried from call to call and kept across ``generate`` calls until
``clear()`` (multi-turn use, chat.py:100-111).
"""
import sys

import torch


class GreedySearch:
    def __init__(self, model, tokenizer):
        model.eval()
        self.model = model
        self.tokenizer = tokenizer
        self.past_kv = None

    def clear(self):
        self.past_kv = None

    def _device(self):
        try:
            return next(self.model.parameters()).device
        except (StopIteration, AttributeError, TypeError):
            return torch.device("cuda" if torch.cuda.is_available() else "cpu")

    def _process_texts(self, input_text):
        ids = self.tokenizer.encode(input_text)
        as_row = lambda values: torch.tensor(values).int().unsqueeze(0).to(self._device())
        return {"input_ids": as_row(ids), "attention_mask": as_row([1] * len(ids))}

    def generate(self, text=None, input_ids=None, **kwargs):
        if input_ids is None:
            input_ids = self._process_texts(text)["input_ids"]
        with torch.inference_mode():
            return self._decode(input_ids, **kwargs)

    def _step(self, ids, mask, past):
        out = self.model(input_ids=ids, attention_mask=mask, use_cache=True, return_dict=True, past_key_values=past)
        return out.logits, out.past_key_values

    def _decode(self, input_ids, max_length=100, extra_end_token_ids=[], chunk_size: int = 4096, output=False):
        if input_ids.dim() == 1:
            input_ids = input_ids[None, :]
        input_ids = input_ids.to(self._device())
        assert input_ids.size(0) == 1
        mask = torch.ones_like(input_ids)
        prompt_len = input_ids.size(1)
        stop_ids = list(extra_end_token_ids) + [self.tokenizer.eos_token_id]
        past = self.past_kv
        shown = ""

        for step in range(max_length + 1):
            if step == 0:                                   # prefill: all but the last token in chunks, then the last one
                body = prompt_len - 1
                piece = body if chunk_size is None else chunk_size
                for st in range(0, body, max(piece, 1)):
                    ed = min(body, st + piece)
                    _, past = self._step(input_ids[:, st:ed], mask[:, :ed], past)
            logits, past = self._step(input_ids[:, -1:], mask, past)
            word = logits[:, -1, :].argmax(dim=-1)
            if word.item() in stop_ids or step == max_length:
                break
            input_ids = torch.cat((input_ids, word.view(1, 1).to(input_ids.dtype)), dim=-1)
            mask = torch.cat((mask, torch.ones((1, 1), dtype=mask.dtype, device=mask.device)), dim=-1)
            if output:
                text = self.tokenizer.decode(input_ids.squeeze(0)[prompt_len:])
                if len(text) > len(shown):
                    sys.stdout.write(text[len(shown):])
                    sys.stdout.flush()
                    shown = text

        self.past_kv = past
        if output:
            sys.stdout.write("\n")
            sys.stdout.flush()
        return [self.tokenizer.decode(input_ids.squeeze(0)[prompt_len:])]
