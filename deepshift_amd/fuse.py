"""Inference-time fusion around shift convolutions (no counterpart in the reference, which leaves
BatchNorm / ReLU / residual adds as separate PyTorch ops around ``Conv2dShift``).

``fuse_conv_epilogues(model, example_input)`` traces the model with ``torch.fx`` and rewrites

    Conv2dShift -> BatchNorm2d (eval) [-> + residual] [-> ReLU]

into one :class:`FusedConv2dShift` call: the int32 result of the shift kernel is converted to float,
scaled and shifted per channel (the folded BatchNorm), added to the residual and clamped at zero
in a single pass (``ds_dequantize_affine_i32_f32``) instead of four.  The shift arithmetic itself
is untouched; the float glue differs from the unfused ops by fp32 rounding only.

Where a fused convolution feeds another one (zero padding), the same pass also writes the consumer's
fixed-point input -- rounded to the consumer's I.F grid and zero padded -- so the consumer skips its
own conversion pass, and the float tensor is not written at all when nothing else reads it
(``ds_requantize_affine_pad_i32``).  This is bit-identical to the two passes it replaces.
"""
import operator

import torch
import torch.fx as fx
import torch.nn as nn
import torch.nn.functional as F

from . import kernels, modules, modules_q

__all__ = ["FusedConv2dShift", "FusedLinearShift", "FusedLinearChain", "fuse_conv_epilogues"]

_SHIFT_CONVS = (modules.Conv2dShift, modules_q.Conv2dShiftQ)
_SHIFT_LINEARS = (modules.LinearShift, modules_q.LinearShiftQ)
_SHIFT_LEAVES = _SHIFT_CONVS + _SHIFT_LINEARS


class FusedLinearShift(nn.Module):
    """A kernel-mode LinearShift / LinearShiftQ layer with the ReLU that follows it (mnist.py:36-38): the
    one-launch kernel applies it to its output."""

    def __init__(self, linear):
        super().__init__()
        self.linear = linear

    def forward(self, input):
        if not self.linear.use_kernel:
            return torch.relu(self.linear(input))
        return self.linear._kernel_forward(input, relu=True)


class FusedLinearChain(nn.Module):
    """Kernel-mode LinearShift / LinearShiftQ layers that feed each other directly, each optionally followed by
    a ReLU -- the shape of the MNIST MLP, mnist.py:23-39 -- in one call of the library
    (``kernels.linear_chain``): ONE launch where that is the faster way (narrow layers, whose persistent
    grid is small enough for its barriers to cost less than the launches they save), else a launch per
    layer issued inside the call (the 512-wide MNIST MLP at batch 64 takes 50 us as one launch, 39 us as
    three).  Bit-identical to the layers run one by one from Python, which is what happens where the
    library has no such form: layers of different field widths or activation formats, a layer too large
    for the one-launch kernel, host execution."""

    def __init__(self, linears, relus):
        super().__init__()
        self.linears = nn.ModuleList(linears)
        self.relus = [bool(r) for r in relus]
        self.force = False   # True: the one-launch form whatever the size (tests, measurements)

    def _one_by_one(self, input):
        x = input
        for linear, relu in zip(self.linears, self.relus):
            if linear.use_kernel:
                x = linear._kernel_forward(x, relu=relu)
            else:
                x = torch.relu(linear(x)) if relu else linear(x)
        return x

    def forward(self, input):
        first = self.linears[0]
        kind = type(first)
        I, Fb = first.act_integer_bits, first.act_fraction_bits
        if not all(type(m) is kind and m.use_kernel and m.use_cuda and
                   (m.act_integer_bits, m.act_fraction_bits) == (I, Fb) for m in self.linears):
            return self._one_by_one(input)
        lead = input.shape[:-1]
        x2d = input.reshape(-1, first.in_features).float()
        M = x2d.shape[0]
        if not x2d.is_cuda or not all(kernels.small_linear_serves(M, m.in_features, m.out_features)
                                      for m in self.linears):
            return self._one_by_one(input)
        round_to_fixed = isinstance(first, modules_q.LinearShiftQ)   # modules_q.py:115-125 / modules.py:24-31
        layers = []
        for m, relu in zip(self.linears, self.relus):
            cw = m.packed_weights()
            bias = m._fixed_bias.get(m.bias, I, Fb, round_to_fixed=round_to_fixed)
            layers.append((kernels._tiled_of(cw, m.out_features, m.in_features), bias, m.in_features,
                           m.out_features, kernels.kernel_bits(cw), cw.base, relu))
        cache = self.__dict__.setdefault("_chain_workspace", {})
        out = kernels.linear_chain(x2d, layers, I, Fb, round_to_fixed, cache, "one" if self.force else None)
        if out is None:
            return self._one_by_one(input)
        return out.reshape(*lead, self.linears[-1].out_features)

    def status(self):
        """0, or the number of the barrier at which a launch gave up waiting for the grid to be resident (its
        result was undefined); synchronises with the device."""
        return kernels.linear_chain_status(self.__dict__.get("_chain_workspace", {}))

    def __getstate__(self):
        state = self.__dict__.copy()
        state.pop("_chain_workspace", None)
        return state


class FusedConv2dShift(nn.Module):
    """A kernel-mode shift convolution with its BatchNorm folded into the dequantisation pass,
    optionally followed by a residual add and ReLU."""

    def __init__(self, conv, bn=None, relu=False):
        super().__init__()
        self.conv = conv
        self.relu = relu
        self.prequantized = False  # the input is this layer's int32 padded input, made by its producer
        self.input_nonneg = False  # ... and that producer ends in a ReLU
        self.emit = None           # (padding, I, F, want_float, dtype) of the consumers' input to produce
        self.pool = None           # (kernel, stride, padding) of a max pooling that follows the ReLU
        if bn is not None:
            if bn.training or not bn.track_running_stats:
                raise ValueError("only an eval-mode BatchNorm with running statistics can be folded")
            var, mean = bn.running_var.detach().float(), bn.running_mean.detach().float()
            weight = bn.weight.detach().float() if bn.affine else torch.ones_like(var)
            bias = bn.bias.detach().float() if bn.affine else torch.zeros_like(var)
            scale = weight / torch.sqrt(var + bn.eps)
            self.register_buffer("scale", scale.contiguous())
            self.register_buffer("shift", (bias - mean * scale).contiguous())
        else:
            self.scale = None
            self.shift = None

    def _check_handoff_dtype(self, input, conc_weight):
        """The producer's pass writes this layer's input in the dtype chosen when the model was fused;
        weights repacked since (``load_state_dict``) may need the other kernel."""
        if not self.prequantized:
            return
        conv = self.conv
        paired = kernels.paired_fields(conc_weight, conv.out_channels, conv.act_integer_bits,
                                       conv.act_fraction_bits)
        if (input.dtype == torch.int8) != bool(paired):
            raise RuntimeError("the weights of a fused shift convolution changed in a way that moves it "
                               "between the int8 and int32 kernels; fuse the model again")

    def forward(self, input, residual=None):
        conv = self.conv
        conc_weight = conv.packed_weights()
        self._check_handoff_dtype(input, conc_weight)
        return modules.conv_kernel_forward(conv, input, conc_weight, self.scale, self.shift,
                                           residual, self.relu, self.prequantized, self.emit, self.pool,
                                           self.input_nonneg)


class FusedShortcutPair(nn.Module):
    """A residual block's first convolution and its 1 x 1 shortcut, both fused convolutions over the same
    tensor with the same stride, run as ONE launch (``kernels.conv2d_tiled_fused_pair``): the shortcut
    reads the centre taps of the padded fixed-point input that was made for the first convolution, so
    it needs neither a conversion pass of its own nor the float form of the block's input.  Returns
    ``(result of the first, result of the shortcut)``, each what the module by itself would return."""

    def __init__(self, first, shortcut):
        super().__init__()
        self.first = first
        self.shortcut = shortcut

    @staticmethod
    def _spec(fused, conc_weight, crop, residual):
        conv = fused.conv
        spec = dict(tiled=kernels._tiled_of(conc_weight, conv.out_channels, conv.in_channels, *conv.kernel_size),
                    bias=conv._fixed_bias.get(conv.bias, conv.act_integer_bits, conv.act_fraction_bits,
                                              round_to_fixed=True),
                    O=conv.out_channels, kernel_size=conv.kernel_size, crop=crop,
                    bits=kernels.kernel_bits(conc_weight), scale=fused.scale, shift=fused.shift,
                    residual=residual, relu=fused.relu, want_float=True,
                    q_cache=conv.__dict__.setdefault("_handoff_buffers", {}))
        if fused.emit is not None:
            padding, I, Fq, want_float = fused.emit[:4]
            spec["emit"] = (padding, I, Fq, fused.emit[4] if len(fused.emit) == 5 else torch.int32)
            spec["want_float"] = want_float
        return spec

    @staticmethod
    def _result(fused, out, q):
        if fused.emit is None:
            return out
        return (out, q) if fused.emit[3] else q

    def forward(self, xq, residual_first=None, residual_shortcut=None):
        a, b = self.first, self.shortcut
        cwa, cwb = a.conv.packed_weights(), b.conv.packed_weights()
        if not _pairable_weights(cwa, cwb) or xq.dtype != torch.int32:
            raise RuntimeError("the weights of a paired shortcut changed in a way that needs another kernel; "
                               "fuse the model again")
        (oa, qa), (ob, qb) = kernels.conv2d_tiled_fused_pair(
            xq, a.conv.stride, a.conv.act_fraction_bits,
            self._spec(a, cwa, (0, 0), residual_first), self._spec(b, cwb, tuple(a.conv.padding), residual_shortcut))
        return self._result(a, oa, qa), self._result(b, ob, qb)


def _pairable_weights(cwa, cwb):
    """Both layers run the same form of the shift-plane kernel: fields of the same width (at most 4
    bits), no base, no ternary blob, the same "top value unused" flag."""
    if cwa is None or cwb is None or cwa.base != 0 or cwb.base != 0:
        return False
    ka, kb = kernels.kernel_bits(cwa), kernels.kernel_bits(cwb)
    from . import _lib
    if (ka | kb) & _lib.DS_BITS_ZERO_TOP:
        return False
    return ka == kb and (ka & 0xff) <= 4


class _Tracer(fx.Tracer):
    def is_leaf_module(self, m, qualname):
        return isinstance(m, _SHIFT_LEAVES) or super().is_leaf_module(m, qualname)


def _is_relu(node, mods):
    if node.op == "call_function" and node.target in (F.relu, torch.relu):
        return True
    if node.op == "call_method" and node.target in ("relu", "relu_"):
        return True
    return node.op == "call_module" and isinstance(mods.get(node.target), nn.ReLU)


def _square(v):
    if isinstance(v, (tuple, list)):
        return int(v[0]) if len(v) == 1 or (len(v) == 2 and v[0] == v[1]) else None
    return int(v) if isinstance(v, int) else None


def _max_pool_of(node, mods):
    """(kernel, stride, padding) if ``node`` is a plain square 2-D max pooling, else None."""
    if node.op == "call_module" and isinstance(mods.get(node.target), nn.MaxPool2d):
        m = mods[node.target]
        spec = dict(kernel_size=m.kernel_size, stride=m.stride, padding=m.padding, dilation=m.dilation,
                    ceil_mode=m.ceil_mode, return_indices=m.return_indices)
    elif node.op == "call_function" and node.target is F.max_pool2d:
        names = ("kernel_size", "stride", "padding", "dilation", "ceil_mode", "return_indices")
        spec = dict(stride=None, padding=0, dilation=1, ceil_mode=False, return_indices=False)
        spec.update(zip(names, node.args[1:]))
        spec.update(node.kwargs)
        if "kernel_size" not in spec:
            return None
    else:
        return None
    if spec["ceil_mode"] or spec["return_indices"] or _square(spec["dilation"]) != 1:
        return None
    k = _square(spec["kernel_size"])
    st = k if spec["stride"] in (None, ()) else _square(spec["stride"])
    pd = _square(spec["padding"])
    if k is None or st is None or pd is None or 2 * pd > k:
        return None
    return (k, st, pd)


def _is_add(node):
    return (node.op == "call_function" and node.target in (operator.add, torch.add, operator.iadd)
            and len(node.args) == 2 and not node.kwargs
            and all(isinstance(a, fx.Node) for a in node.args))


def _sole_user(node):
    users = list(node.users)
    return users[0] if len(users) == 1 else None


def fuse_conv_epilogues(model, handoff=True):
    """Return a ``torch.fx.GraphModule`` equivalent to ``model`` (eval mode) with every kernel-mode
    shift convolution fused with the BatchNorm / residual add / ReLU that consume its output, and every
    kernel-mode shift linear layer with its ReLU.
    ``handoff``: fused convolutions that feed each other pass the fixed-point tensor directly."""
    model.eval()
    graph = _Tracer().trace(model)
    gm = fx.GraphModule(model, graph)
    mods = dict(gm.named_modules())
    count = 0
    for node in list(gm.graph.nodes):
        if node.op != "call_module":
            continue
        conv = mods.get(node.target)
        if isinstance(conv, _SHIFT_LINEARS) and conv.use_kernel:
            # a fully connected layer and its ReLU
            nxt = _sole_user(node)
            if nxt is not None and _is_relu(nxt, mods):
                name = "fused_%d" % count
                count += 1
                gm.add_module(name, FusedLinearShift(conv))
                with gm.graph.inserting_after(nxt):
                    new = gm.graph.call_module(name, (node.args[0],))
                nxt.replace_all_uses_with(new)
                gm.graph.erase_node(nxt)
                gm.graph.erase_node(node)
            continue
        if not isinstance(conv, _SHIFT_CONVS) or not conv.use_kernel:
            continue
        chain = [node]
        bn = None
        nxt = _sole_user(chain[-1])
        if nxt is not None and nxt.op == "call_module" and isinstance(mods.get(nxt.target), nn.BatchNorm2d):
            bn = mods[nxt.target]
            chain.append(nxt)
            nxt = _sole_user(nxt)
        residual = None
        if nxt is not None and _is_add(nxt):
            other = nxt.args[1] if nxt.args[0] is chain[-1] else nxt.args[0]
            # the fused call is emitted at the position of the last fused node, where the other
            # operand of the add already exists
            if other is not chain[-1]:
                residual = other
                chain.append(nxt)
                nxt = _sole_user(nxt)
        relu = False
        if nxt is not None and _is_relu(nxt, mods):
            relu = True
            chain.append(nxt)
            nxt = _sole_user(nxt)
        pool = None
        if nxt is not None and residual is None and len(chain) > 1 and nxt.args and nxt.args[0] is chain[-1]:
            pool = _max_pool_of(nxt, mods)
            if pool is not None:
                chain.append(nxt)
        if len(chain) == 1:
            continue  # nothing to fuse
        name = "fused_%d" % count
        count += 1
        gm.add_module(name, FusedConv2dShift(conv, bn, relu))
        gm.get_submodule(name).pool = pool
        with gm.graph.inserting_after(chain[-1]):
            args = (node.args[0],) if residual is None else (node.args[0], residual)
            new = gm.graph.call_module(name, args)
        chain[-1].replace_all_uses_with(new)
        for old in reversed(chain):
            gm.graph.erase_node(old)
    if handoff:
        _hand_off_fixed_point(gm)
        _pair_shortcuts(gm)
    _chain_linears(gm)
    gm.graph.lint()
    gm.recompile()
    return gm


def _chain_linears(gm):
    """Kernel-mode linear layers (with or without their fused ReLU) that feed each other directly become one
    :class:`FusedLinearChain` (two to four layers per chain)."""
    mods = dict(gm.named_modules())

    def linear_of(n):
        """(LinearShift module, relu) if node ``n`` is a kernel-mode linear layer call, else None."""
        m = mods.get(n.target) if n.op == "call_module" else None
        if isinstance(m, FusedLinearShift) and m.linear.use_kernel:
            return m.linear, True
        if isinstance(m, _SHIFT_LINEARS) and m.use_kernel:
            return m, False
        return None

    count = 0
    taken = set()
    for node in list(gm.graph.nodes):
        if node in taken or linear_of(node) is None or len(node.args) != 1 or node.kwargs:
            continue
        chain = [node]
        while len(chain) < 4:
            nxt = _sole_user(chain[-1])
            if nxt is None or linear_of(nxt) is None or tuple(nxt.args) != (chain[-1],) or nxt.kwargs:
                break
            if linear_of(nxt)[0].in_features != linear_of(chain[-1])[0].out_features:
                break
            chain.append(nxt)
        if len(chain) < 2:
            continue
        taken.update(chain)
        pairs = [linear_of(n) for n in chain]
        name = "chain_%d" % count
        count += 1
        gm.add_module(name, FusedLinearChain([m for m, _ in pairs], [r for _, r in pairs]))
        with gm.graph.inserting_after(chain[-1]):
            new = gm.graph.call_module(name, (chain[0].args[0],))
        chain[-1].replace_all_uses_with(new)
        for old in reversed(chain):
            gm.graph.erase_node(old)
    return count


def _input_key(conv):
    """What a kernel-mode convolution needs of its fixed-point input -- (padding, I, F, dtype) -- or
    None if it pads by itself."""
    if conv.padding_mode != 'zeros' or not conv.use_kernel:
        return None
    param = conv.weight if isinstance(conv, modules_q.Conv2dShiftQ) else conv.shift
    conc_weight = conv.packed_weights() if param.is_cuda else conv.conc_weight
    paired = kernels.paired_fields(conc_weight, conv.out_channels, conv.act_integer_bits,
                                   conv.act_fraction_bits)
    return (tuple(conv.padding), conv.act_integer_bits, conv.act_fraction_bits,
            torch.int8 if paired else torch.int32)


def _hand_off_fixed_point(gm):
    """Second pass: a fused convolution whose result feeds fused convolutions also writes their
    fixed-point padded input, and they read that instead of converting the float tensor again."""
    mods = dict(gm.named_modules())

    def fused(n):
        m = mods.get(n.target) if n.op == "call_module" else None
        return m if isinstance(m, FusedConv2dShift) else None

    for node in list(gm.graph.nodes):
        producer = fused(node)
        if producer is None or producer.emit is not None:
            continue
        key, takers = None, []
        for user in node.users:
            consumer = fused(user)
            if consumer is None or user.args[0] is not node or consumer.prequantized:
                continue
            k = _input_key(consumer.conv)
            if k is None or (key is not None and k != key):
                continue
            key = k
            takers.append(user)
        if not takers:
            continue
        # the float result is still needed by any other use, including a taker's residual operand
        want_float = any(u not in takers or node in u.args[1:] for u in node.users)
        producer.emit = key[:3] + (want_float, key[3])
        if want_float:
            with gm.graph.inserting_after(node):
                q = gm.graph.call_function(operator.getitem, (node, 1))
                f = gm.graph.call_function(operator.getitem, (node, 0))
            node.replace_all_uses_with(f, delete_user_cb=lambda u: u is not f and u is not q)
        else:
            q = node
        for user in takers:
            user.args = (q,) + tuple(user.args[1:])
            fused(user).prequantized = True
            fused(user).input_nonneg = bool(producer.relu)


def _pair_shortcuts(gm):
    """Third pass: where a fused k x k convolution A reads the fixed-point tensor its producer P made for
    it, and a fused 1 x 1 convolution B with the same stride and no padding reads P's float result -- the
    two branches of a down-sampling residual block -- run A and B as one launch on P's fixed-point tensor
    (B reads the centre taps: the padded tensor cropped by A's padding).  If nothing else reads P's
    float result it is no longer written."""
    mods = dict(gm.named_modules())

    def fused(n):
        m = mods.get(n.target) if n.op == "call_module" else None
        return m if isinstance(m, FusedConv2dShift) else None

    count = 0
    for node in list(gm.graph.nodes):
        A = fused(node)
        if A is None or not A.prequantized or A.pool is not None:
            continue
        q_node = node.args[0]
        if q_node.op == "call_function" and q_node.target is operator.getitem and q_node.args[1] == 1:
            producer, f_nodes = q_node.args[0], [u for u in q_node.args[0].users
                                                 if u.op == "call_function" and u.target is operator.getitem
                                                 and u.args[1] == 0]
        else:
            continue   # the producer writes no float result: nobody reads the block input as float
        ca = A.conv
        for f_node in f_nodes:
            for user in list(f_node.users):
                B = fused(user)
                if B is None or user.args[0] is not f_node or B.prequantized or B.pool is not None:
                    continue
                cb = B.conv
                if (tuple(cb.kernel_size) != (1, 1) or tuple(cb.padding) != (0, 0) or cb.padding_mode != 'zeros'
                        or tuple(cb.stride) != tuple(ca.stride) or cb.in_channels != ca.in_channels
                        or ca.padding_mode != 'zeros'
                        or (cb.act_integer_bits, cb.act_fraction_bits) != (ca.act_integer_bits, ca.act_fraction_bits)
                        or ca.out_channels % 64 or cb.out_channels % 64
                        or tuple(ca.kernel_size) != (2 * ca.padding[0] + 1, 2 * ca.padding[1] + 1)):
                    continue
                param = ca.shift if hasattr(ca, "shift") else ca.weight
                if not param.is_cuda or not _pairable_weights(ca.packed_weights(), cb.packed_weights()):
                    continue
                if kernels.paired_fields(ca.packed_weights(), ca.out_channels, ca.act_integer_bits,
                                         ca.act_fraction_bits):
                    continue   # int8 activations: another kernel
                # the pair runs where the earlier of the two stands (the users of both come later), so
                # every operand must exist by then
                order = {n: i for i, n in enumerate(gm.graph.nodes)}
                earlier = node if order[node] < order[user] else user
                operands = [q_node] + [a for a in list(node.args[1:]) + list(user.args[1:]) if isinstance(a, fx.Node)]
                if any(order[a] > order[earlier] for a in operands):
                    continue
                name = "pair_%d" % count
                count += 1
                gm.add_module(name, FusedShortcutPair(A, B))
                res_a = node.args[1] if len(node.args) > 1 else None
                res_b = user.args[1] if len(user.args) > 1 else None
                with gm.graph.inserting_before(earlier):
                    both = gm.graph.call_module(name, (q_node, res_a, res_b))
                with gm.graph.inserting_after(both):
                    out_b = gm.graph.call_function(operator.getitem, (both, 1))
                    out_a = gm.graph.call_function(operator.getitem, (both, 0))
                node.replace_all_uses_with(out_a)
                user.replace_all_uses_with(out_b)
                gm.graph.erase_node(node)
                gm.graph.erase_node(user)
                # P's float result: still written only if something else reads it
                if not f_node.users:
                    P = fused(producer)
                    gm.graph.erase_node(f_node)
                    if P is not None and P.emit is not None and not any(
                            u.op == "call_function" and u.target is operator.getitem and u.args[1] == 0
                            for u in producer.users):
                        P.emit = P.emit[:3] + (False,) + P.emit[4:]
                        q_node.replace_all_uses_with(producer)
                        gm.graph.erase_node(q_node)
                break
            else:
                continue
            break
    return count
