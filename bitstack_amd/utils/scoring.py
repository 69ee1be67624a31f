"""Importance scoring of the residual blocks and generation of the memory-sorted list of
compression configs, driven by the library's forwards.

What the reference does in `bitstack/main.py:138-166` (perplexity of a calibration set with
one linear at a time given one more block) and `:168-187` with
`bitstack/utils/model_utils.py:26-66` (`sort_layers_and_bits_average`, `generate_configs`)
and `:117-133` (`eval_ppl`).  The calibration tokens are the caller's (there is no dataset
loader here); the model is a `SyntheticLlamaDecoder` (random-init or read from a
reference-format checkpoint), whose `prefill(..., all_logits=True)` is the full-sequence
forward."""
from __future__ import annotations

import json
import math
import os

import torch
import torch.nn.functional as F


def _batches(decoder, input_ids):
    """[(ids [B, n] on the device, number of real rows)]: the last batch is padded by repeating rows."""
    B = decoder.batch
    out = []
    for i in range(0, input_ids.shape[0], B):
        ids = input_ids[i:i + B].to(decoder.dev)
        real = ids.shape[0]
        if real < B:
            ids = torch.cat([ids, ids[-1:].expand(B - real, -1)])
        out.append((ids, real))
    return out


def _nll(logits, ids, real):
    """Mean next-token negative log-likelihood per sequence (fp32 log-softmax, one sequence at a
    time so that the fp32 copy of the logits stays small)."""
    out = []
    for b in range(real):
        loss = F.cross_entropy(logits[b, :-1].float(), ids[b, 1:], reduction="none")
        out.append(loss.mean())
    return torch.stack(out)


@torch.no_grad()
def eval_ppl(decoder, input_ids: torch.Tensor) -> float:
    """exp(mean over sequences of the mean next-token negative log-likelihood), as
    model_utils.py:117-133.  `input_ids` is [n_sequences, seqlen]; sequences are run in
    batches of the decoder's batch size."""
    nlls = [_nll(decoder.prefill(ids, all_logits=True), ids, real) for ids, real in _batches(decoder, input_ids)]
    return float(torch.exp(torch.cat(nlls).mean()))


def all_linears(decoder):
    """The decoder's BitStackLinear modules in model order, as (name, module)."""
    out = []
    for L, row in enumerate(decoder.lin):
        for p, m in row.items():
            out.append((getattr(m, "name", None) or f"layer.{L}.{p}", m))
    return out


def all_linears_with_layer(decoder):
    out = []
    for L, row in enumerate(decoder.lin):
        for p, m in row.items():
            out.append((getattr(m, "name", None) or f"layer.{L}.{p}", m, L))
    return out


@torch.no_grad()
def score_importance(decoder, input_ids: torch.Tensor, niter: int, progress=None, reuse_prefix=True):
    """For bit = 1 .. niter - 1: every linear at `bit` blocks, then one linear at a time at
    bit + 1 and the calibration perplexity with it (main.py:146-157).  Returns the dict the
    reference writes to reduced_ppl_average.json.  The block counts are restored.

    reuse_prefix: a linear of decoder layer L changes nothing before layer L, so per bit
    level the input of every layer is kept from one run at the level's block counts and each
    evaluation resumes at its linear's layer - the same numbers for about half the work
    (batches x layers x batch x seqlen x hidden fp16 values are held meanwhile)."""
    linears = all_linears_with_layer(decoder)
    saved = [m.w_bit for _, m, _ in linears]
    batches = _batches(decoder, input_ids)
    try:
        original = eval_ppl(decoder, input_ids)
        ppls = []
        for bit in range(1, niter):
            for _, m, _ in linears:
                m.set_bit(bit)
            kept = []
            if reuse_prefix:
                for ids, _ in batches:
                    keep = []
                    decoder.prefill(ids, keep=keep)
                    kept.append(keep)
            per_bit = []
            for name, m, L in linears:
                m.set_bit(bit + 1)
                if reuse_prefix:
                    nlls = [_nll(decoder.prefill(ids, all_logits=True, first_layer=L, hidden=kept[b][L] if L else None), ids, real)
                            for b, (ids, real) in enumerate(batches)]
                    ppl = float(torch.exp(torch.cat(nlls).mean()))
                else:
                    ppl = eval_ppl(decoder, input_ids)
                m.set_bit(bit)
                per_bit.append({"layer": name, "ppl": ppl})
                if progress is not None:
                    progress(bit, name, ppl)
            ppls.append({"bit": bit, "ppls": per_bit})
            del kept
        return {"original_ppl": original, "reduced_ppl": ppls}
    finally:
        for (_, m, _), b in zip(linears, saved):
            m.set_bit(b)


def _is_nan(v) -> bool:
    return isinstance(v, float) and math.isnan(v) or str(v).lower() == "nan"


def sort_layers_and_bits_average(data):
    """Order in which blocks are added: bit level by bit level, within a level the linear
    whose extra block lowers the perplexity most first (model_utils.py:26-51).  A NaN
    perplexity is replaced by that linear's perplexity at the next level plus the level's
    largest finite one (so it sorts last, in next-level order; plus 0 when the level's first
    entry is the NaN, as the reference's max() then yields NaN); a NaN at the last level is an error."""
    levels = [[dict(e) for e in lvl["ppls"]] for lvl in data["reduced_ppl"]]
    for b in reversed(range(len(levels))):
        finite = [e["ppl"] for e in levels[b] if not _is_nan(e["ppl"])]
        # the reference takes Python's max() over the level: that is the largest finite value,
        # unless the level's FIRST entry is NaN (every comparison with it fails), and then 0
        top = 0 if (_is_nan(levels[b][0]["ppl"]) or not finite) else max(finite)
        for idx, e in enumerate(levels[b]):
            if _is_nan(e["ppl"]):
                if b == len(levels) - 1:
                    raise ValueError("Last bit is nan")
                nxt = levels[b + 1][idx]
                assert nxt["layer"] == e["layer"]
                e["ppl"] = nxt["ppl"] + top
    order = []
    for lvl in levels:
        order.extend(e["layer"] for e in sorted(lvl, key=lambda e: e["ppl"]))
    return order


def generate_configs(sorted_layer_bits, memory_per_bit, total_memory):
    """[{memory, layers}]: every linear at one block, then one more block at a time in the
    given order, memory growing by that linear's bytes per block (model_utils.py:53-66)."""
    layers = {name: 1 for name in memory_per_bit}
    configs = [{"memory": total_memory, "layers": dict(layers)}]
    for name in sorted_layer_bits:
        total_memory += memory_per_bit[name]
        layers[name] += 1
        configs.append({"memory": total_memory, "layers": dict(layers)})
    return configs


def compression_configs_for(decoder, reduced_ppls):
    """The list main.py:168-187 writes to compression_config.json: memory counts one block of
    every linear plus everything that is not a compressed linear (embedding, lm_head, norms)."""
    linears = all_linears(decoder)
    per_bit = {name: int(m.memory_per_bit()) for name, m in linears}
    extra = (decoder.embed.numel() + decoder.lm_head.numel() + decoder.norm_w.numel() + decoder.final_norm.numel()) * 2
    for _, m in linears:
        if getattr(m, "bias", None) is not None:
            extra += m.bias.numel() * m.bias.element_size()
    return generate_configs(sort_layers_and_bits_average(reduced_ppls), per_bit, sum(per_bit.values()) + extra)


def save_scores_and_configs(path, reduced_ppls, configs):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "reduced_ppl_average.json"), "w") as f:
        json.dump(reduced_ppls, f, indent=4)
    with open(os.path.join(path, "compression_config.json"), "w") as f:
        json.dump(configs, f, indent=4)
