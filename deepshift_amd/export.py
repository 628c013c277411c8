"""Packed-weight export file: the sign+shift words of every kernel-mode shift layer of a model,
so that deployment loads 5-bit codes instead of float ``shift`` / ``sign`` parameters.

No counterpart in the reference, whose checkpoints hold the float parameters and re-pack them on
the first forward (modules.py:25-27, 153-155).  The file is a plain ``torch.save`` of tensors,
ints and strings and loads with ``torch.load(..., weights_only=True)``.
"""
import torch

from . import modules, modules_q, utils

FORMAT = "deepshift-packed-v1"
_SHIFT_TYPES = (modules.LinearShift, modules.Conv2dShift, modules_q.LinearShiftQ, modules_q.Conv2dShiftQ)


def _shift_layers(model):
    return [(name, m) for name, m in model.named_modules() if isinstance(m, _SHIFT_TYPES)]


def _pack(m):
    return m.packed_weights()


def _scan_fields(words, N, K, bits):
    """(largest field below 32 or -1, number of zero codes) of reference-format words, counted on the
    device."""
    from . import _lib
    out = torch.empty(4, dtype=torch.int32, device=words.device)
    _lib.call("ds_scan_words_i32", _lib.ptr(words), N, K, bits, _lib.ptr(out), _lib.current_stream(words.device))
    top, zeros = out[:2].tolist()
    return int(top), int(zeros)


def packed_state(model):
    """``{"format", "layers": {name: {"words", "bits", "base", "shape", "bias"}}}`` of a converted
    model (packing happens on the GPU, so the model's shift layers must live there)."""
    layers = {}
    for name, m in _shift_layers(model):
        cw = _pack(m)
        shape = list((m.shift if hasattr(m, "shift") else m.weight).shape)
        entry = {"words": cw.data.detach().cpu(), "bits": int(cw.bits), "base": int(cw.base), "shape": shape,
                 "zero_top_bits": int(getattr(cw, "zero_top_bits", 0))}
        if getattr(cw, "max_field", None) is not None:
            entry["max_field"] = int(cw.max_field)  # lets the loader pick the kernel form without the top plane
        if m.bias is not None:
            entry["bias"] = m.bias.detach().float().cpu()
        layers[name] = entry
    return {"format": FORMAT, "layers": layers}


def save_packed(model, path):
    torch.save(packed_state(model), path)


def load_packed(model, path_or_state, device=None):
    """Install the packed words of an export file into ``model``'s shift layers (matched by module
    name and weight shape) and switch them to the kernel path.  Returns the number of layers set."""
    state = path_or_state
    if not isinstance(state, dict):
        state = torch.load(path_or_state, map_location="cpu", weights_only=True)
    if state.get("format") != FORMAT:
        raise ValueError("not a %s file" % FORMAT)
    found = dict(_shift_layers(model))
    missing = sorted(set(found) - set(state["layers"]))
    extra = sorted(set(state["layers"]) - set(found))
    if missing or extra:
        raise KeyError("layers without packed weights: %s; packed weights without a layer: %s" % (missing, extra))
    for name, entry in state["layers"].items():
        m = found[name]
        param = m.shift if hasattr(m, "shift") else m.weight
        if list(param.shape) != list(entry["shape"]):
            raise ValueError("%s: packed for shape %s, layer has %s" % (name, entry["shape"], list(param.shape)))
        dev = device or param.device
        if torch.device(dev).type != "cuda":
            raise ValueError("packed weights are consumed by the GPU kernels: move the model to the GPU first")
        bits, base = int(entry["bits"]), int(entry["base"])
        K = param[0].numel()
        comm = (K + 32 // (bits + 1) - 1) // (32 // (bits + 1))
        words = entry["words"].to(dev, torch.int32).contiguous()
        if words.numel() != param.shape[0] * comm:
            raise ValueError("%s: %d packed words, expected %d" % (name, words.numel(), param.shape[0] * comm))
        # max_field and zero_top_bits select kernel forms that assume them: take them from the words,
        # never from the file (an understated value would give wrong sums without any error)
        top, _ = _scan_fields(words, param.shape[0], K, bits)
        top = max(top, 0)
        zero_top = utils._zero_top_width(top) if (bits == 6 and base == 0) else 0
        for key, mine in (("max_field", top), ("zero_top_bits", zero_top)):
            if key in entry and int(entry[key]) != mine:
                raise ValueError("%s: the file says %s = %s, its words say %d" % (name, key, entry[key], mine))
        m.conc_weight = utils.ConcWeight(words, base, bits, zero_top, top)
        m.use_kernel = True
        if "bias" in entry and m.bias is not None:
            with torch.no_grad():
                m.bias.copy_(entry["bias"].to(m.bias.device))
    return len(state["layers"])
