"""Front end for the reference's text configuration files: a solver prototxt and the network
prototxt it names (src/parser/cnn.proto; read by Parser::read_proto_from_text_file and turned into
bridges by DeepNet::construct_network, src/DeepNet.h:968-2030).

No protobuf runtime is needed: `parse` reads the text format (``key: value``, ``key { ... }``,
``key: { ... }``, ``#`` comments, quoted strings, enum identifiers, numbers, booleans) into nested
messages; `network_from_prototxt` maps a sequential network of the layer types of the LeNet and
CaffeNet/AlexNet definitions onto `nets.LayerSpec` records; `solver_from_prototxt` fills
`cct_solver_param` with the defaults cnn.proto declares.

Rules kept from the reference:
  * layer types are compared case-insensitively (src/DeepNet.h:148, 1026);
  * the first ``Data`` layer of the requested phase gives batch size, crop size and scale
    (src/parser/corpus.h:44-59, 205-232); ``Accuracy`` layers are skipped (src/DeepNet.h:836);
  * ``blobs_lr`` / ``weight_decay`` (old) are read first and ``param { lr_mult decay_mult }`` (new)
    overrides them; absent multipliers are 1 (src/bridges/ParallelizedBridge_impl.hxx:343-361,
    429-447);
  * a layer whose top equals its bottom runs in place (src/DeepNet.h:1055-1060);
  * output sizes: convolution (n + 2p - k)/s + 1, pooling (n - k)/s + 1 unpadded
    (src/DeepNet.h:112-115, 1374-1376);
  * the reference prints a warning and ignores ``group`` (src/DeepNet.h:1075-1077); here
    ``groups="honor"`` (default) runs the grouped convolution the file asks for and
    ``groups="ignore"`` reproduces the reference.
  * a blob read by several layers needs no Split layer in the file (the reference inserts the split
    itself, src/DeepNet.h:1924-2028); an explicit ``Split`` layer is accepted and only renames the
    blob; ``Concat`` stacks its bottoms along the channel axis (src/DeepNet.h:1700-1757).
Eltwise / BatchNorm / Scale layers are outside this front end and are rejected with the layer's name
in the message.
"""
import os
import re

from . import _lib, nets
from .bridges import solver_param

__all__ = ["Message", "parse", "parse_file", "solver_from_prototxt", "network_from_prototxt", "NetworkDef",
           "load_solver", "PrototxtError"]


class PrototxtError(ValueError):
    pass


class Message:
    """One parsed message: every field keeps the list of its values in file order."""

    def __init__(self):
        self.fields = {}

    def add(self, key, value):
        self.fields.setdefault(key, []).append(value)

    def has(self, key):
        return key in self.fields

    def all(self, key):
        return list(self.fields.get(key, []))

    def get(self, key, default=None):
        """Last value, as protobuf's text parser keeps for an optional field given twice."""
        v = self.fields.get(key)
        return v[-1] if v else default

    def msg(self, key):
        """Sub-message `key`, or an empty message when absent (so defaults apply)."""
        v = self.get(key)
        if v is None:
            return Message()
        if not isinstance(v, Message):
            raise PrototxtError("field %r is not a message" % key)
        return v

    def __repr__(self):
        return "Message(%r)" % (self.fields,)


_TOKEN = re.compile(r"""
    \s+ | \#[^\n]* |                                   # blanks, comments
    (?P<str>"(?:[^"\\]|\\.)*" | '(?:[^'\\]|\\.)*') |
    (?P<punct>[{}:<>;,\[\]]) |
    (?P<atom>[^\s{}:<>;,\[\]"'\#]+)
""", re.X)

_ESCAPES = {"n": "\n", "t": "\t", "r": "\r", "\\": "\\", '"': '"', "'": "'", "0": "\0"}


def _tokens(text):
    pos, out = 0, []
    while pos < len(text):
        m = _TOKEN.match(text, pos)
        if not m:
            line = text.count("\n", 0, pos) + 1
            raise PrototxtError("line %d: cannot read %r" % (line, text[pos:pos + 20]))
        line = text.count("\n", 0, pos) + 1 if (m.lastgroup) else 0
        if m.lastgroup == "str":
            body = m.group("str")[1:-1]
            out.append(("str", re.sub(r"\\(.)", lambda e: _ESCAPES.get(e.group(1), e.group(1)), body), line))
        elif m.lastgroup == "punct":
            out.append(("punct", m.group("punct"), line))
        elif m.lastgroup == "atom":
            out.append(("atom", m.group("atom"), line))
        pos = m.end()
    return out


def _scalar(kind, text):
    if kind == "str":
        return text
    low = text.lower()
    if low == "true":
        return True
    if low == "false":
        return False
    try:
        return int(text, 0)
    except ValueError:
        pass
    try:
        return float(text[:-1] if low.endswith("f") and len(text) > 1 else text)
    except ValueError:
        return text  # enum identifier


def _parse_message(toks, i, closer):
    msg = Message()
    while i < len(toks):
        kind, text, line = toks[i]
        if kind == "punct" and text == closer:
            return msg, i + 1
        if kind == "punct" and text in ";,":
            i += 1
            continue
        if kind != "atom":
            raise PrototxtError("line %d: field name expected, found %r" % (line, text))
        key, i = text, i + 1
        if i >= len(toks):
            raise PrototxtError("line %d: field %r has no value" % (line, key))
        if toks[i][:2] == ("punct", ":"):
            i += 1
            if i >= len(toks):
                raise PrototxtError("line %d: field %r has no value" % (line, key))
        kind, text, line = toks[i]
        if kind == "punct" and text in "{<":
            sub, i = _parse_message(toks, i + 1, "}" if text == "{" else ">")
            msg.add(key, sub)
        elif kind == "punct" and text == "[":
            i += 1
            while i < len(toks) and toks[i][:2] != ("punct", "]"):
                if toks[i][:2] != ("punct", ","):
                    msg.add(key, _scalar(toks[i][0], toks[i][1]))
                i += 1
            i += 1
        elif kind == "punct":
            raise PrototxtError("line %d: value expected for %r, found %r" % (line, key, text))
        else:
            value = _scalar(kind, text)
            i += 1
            # adjacent string literals concatenate
            while kind == "str" and i < len(toks) and toks[i][0] == "str":
                value += toks[i][1]
                i += 1
            msg.add(key, value)
    if closer is not None:
        raise PrototxtError("unbalanced braces: %r expected before the end of the text" % closer)
    return msg, i


def parse(text):
    """Text-format protobuf -> `Message`."""
    msg, _ = _parse_message(_tokens(text), 0, None)
    return msg


def parse_file(path):
    with open(path, "r") as f:
        return parse(f.read())


def _as_message(x):
    return x if isinstance(x, Message) else parse(x)


# ---- solver ------------------------------------------------------------------------------

def solver_from_prototxt(text_or_message):
    """SolverParameter -> (`cct_solver_param`, dict of the fields that steer the training loop:
    net, max_iter, display, snapshot, snapshot_prefix, test_iter, test_interval).  Defaults follow
    src/parser/cnn.proto:56-160: weight_decay 0, regularization_type "L2", display 10 (cnn.proto:104),
    snapshot 0, random_seed -1; momentum, gamma, power, stepsize default to 0 and lr_policy must be
    given (Util::get_learning_rate aborts on an unknown policy, src/util.h:66-93)."""
    m = _as_message(text_or_message)
    policy = m.get("lr_policy")
    if policy is None:
        raise PrototxtError("solver: lr_policy is required")
    if m.get("base_lr") is None:
        raise PrototxtError("solver: base_lr is required")
    sp = solver_param(base_lr=float(m.get("base_lr")), momentum=float(m.get("momentum", 0.0)),
                      gamma=float(m.get("gamma", 0.0)), power=float(m.get("power", 0.0)),
                      weight_decay=float(m.get("weight_decay", 0.0)), stepsize=int(m.get("stepsize", 0)),
                      max_iter=int(m.get("max_iter", 0)), random_seed=int(m.get("random_seed", -1)),
                      lr_policy=str(policy), regularization_type=str(m.get("regularization_type", "L2")))
    control = {
        "net": m.get("net"), "max_iter": int(m.get("max_iter", 0)), "display": int(m.get("display", 10)),
        "snapshot": int(m.get("snapshot", 0)), "snapshot_prefix": m.get("snapshot_prefix"),
        "test_iter": [int(v) for v in m.all("test_iter")], "test_interval": int(m.get("test_interval", 0)),
    }
    return sp, control


# ---- network -----------------------------------------------------------------------------

class NetworkDef:
    """What a network prototxt says once mapped to this library: `layers` (`nets.LayerSpec` list),
    `names` (layer names, same order), and the data layer's `batch_size`, `crop_size`, `scale`,
    `mirror`, `mean_file`, `source` for the chosen phase."""

    def __init__(self):
        self.name = None
        self.layers, self.names = [], []
        self.batch_size = self.crop_size = 0
        self.scale, self.mirror, self.mean_file, self.source = 1.0, False, None, None

    def output_shapes(self, depth, size):
        """[(depth, size)] after every layer for an input of `depth` channels and `size` x `size`."""
        out = []
        in_depth, in_size = depth, size
        for i, s in enumerate(self.layers):
            if s.n_bottoms:
                depth, size = (in_depth, in_size) if s.bottoms[0] < 0 else out[s.bottoms[0]]
            if s.type == nets.CONCAT:
                depth = sum(in_depth if s.bottoms[j] < 0 else out[s.bottoms[j]][0] for j in range(s.n_bottoms))
            if s.type == nets.CONV:
                size = (size + 2 * s.pad - s.kernel_size) // s.stride + 1
                depth = s.num_output
            elif s.type == nets.MAXPOOL:
                size = (size - s.kernel_size) // s.stride + 1
            elif s.type == nets.FC:
                depth, size = s.num_output, 1
            out.append((depth, size))
        return out

    def validate(self, depth, size=None, solver=None, batch=None):
        """Checks the chain against an input of `depth` x `size` x `size` on the host (no device):
        every kernel must fit its (padded) input, groups must divide the depths, and so on.  Raises
        PrototxtError naming the layer as the prototxt does."""
        size = size or self.crop_size
        if not size:
            raise PrototxtError("input size is neither given nor set by crop_size")
        try:
            nets.validate(batch or self.batch_size, depth, size, self.layers, solver)
        except _lib.CctHipError as e:
            msg = str(e)
            hit = re.search(r"layer (\d+): (.*)$", msg)
            if hit:
                raise PrototxtError("layer %r: %s" % (self.names[int(hit.group(1))], hit.group(2))) from None
            raise PrototxtError(msg) from None

    def build(self, depth, size=None, solver=None, batch=None):
        """`nets.Net` on the device; `size` defaults to the data layer's crop size."""
        self.validate(depth, size, solver, batch)
        size = size or self.crop_size
        return nets.Net(batch or self.batch_size, depth, size, self.layers, solver)


_PHASES = {"TRAIN": 0, "TEST": 1, 0: 0, 1: 1}


def _layer_phase(layer):
    """Phase of the layer's first include rule (corpus.h:48 reads include(0).phase()), or None."""
    inc = layer.all("include")
    if not inc:
        return None
    ph = inc[0].get("phase")
    if ph not in _PHASES:
        raise PrototxtError("layer %r: unknown phase %r" % (layer.get("name"), ph))
    return _PHASES[ph]


def _filler(m, what, layer_name):
    t = str(m.get("type", "constant"))
    if t not in nets.FILLER_TYPES:
        raise PrototxtError("layer %r: %s type %r is not supported (constant, xavier, gaussian, bernoulli)"
                            % (layer_name, what, t))
    return nets.filler(t, float(m.get("value", 0.0)), float(m.get("mean", 0.0)), float(m.get("std", 1.0)))


def _multipliers(layer):
    lr, decay = [1.0, 1.0], [1.0, 1.0]
    for i, v in enumerate(layer.all("blobs_lr")[:2]):
        lr[i] = float(v)
    for i, v in enumerate(layer.all("weight_decay")[:2]):
        decay[i] = float(v)
    for i, p in enumerate(layer.all("param")[:2]):
        lr[i] = float(p.get("lr_mult", 1.0))
        decay[i] = float(p.get("decay_mult", 1.0))
    return tuple(lr), tuple(decay)


def network_from_prototxt(text_or_message, phase="TRAIN", groups="honor"):
    """NetParameter -> `NetworkDef`."""
    if groups not in ("honor", "ignore"):
        raise ValueError("groups must be 'honor' or 'ignore'")
    m = _as_message(text_or_message)
    want = _PHASES[phase]
    layers = m.all("layer")
    if m.has("layers"):
        raise PrototxtError("V1 `layers { ... }` definitions are not supported; use `layer { ... }`")
    nd = NetworkDef()
    nd.name = m.get("name")
    data = [l for l in layers if str(l.get("type", "")).upper() == "DATA"]
    chosen = [l for l in data if _layer_phase(l) in (None, want)]
    if not chosen:
        raise PrototxtError("a Data layer is needed (src/DeepNet.h:800-816)")
    d = chosen[0]
    tops = d.all("top")
    if not tops:
        raise PrototxtError("data layer %r has no top" % d.get("name"))
    tp, dp = d.msg("transform_param"), d.msg("data_param")
    nd.batch_size = int(dp.get("batch_size", 0))
    nd.source = dp.get("source")
    nd.crop_size = int(tp.get("crop_size", 0))
    nd.scale = float(tp.get("scale", 1.0))
    nd.mirror = bool(tp.get("mirror", False))
    nd.mean_file = tp.get("mean_file")
    if nd.batch_size <= 0:
        raise PrototxtError("data layer %r: batch_size must be positive" % d.get("name"))

    writer = {tops[0]: -1}     # blob name -> index (in nd.layers) of the layer that wrote it last; -1 = the data layer
    label_blobs = set(tops[1:])
    done_loss = False
    for l in layers:
        name, typ = l.get("name"), str(l.get("type", "")).upper()
        if typ in ("DATA", "ACCURACY"):
            continue
        ph = _layer_phase(l)
        if ph is not None and ph != want:
            continue
        bottoms, tops = l.all("bottom"), l.all("top")
        if done_loss:
            raise PrototxtError("layer %r follows the loss layer" % name)

        def need(cond, what):
            if not cond:
                raise PrototxtError("layer %r: %s" % (name, what))

        def source(blob):
            need(blob in writer, "reads %r, which no earlier layer produces" % blob)
            return writer[blob]
        if typ in ("SOFTMAXWITHLOSS", "SOFTMAX"):
            data_bottoms = [b for b in bottoms if b not in label_blobs]
            need(len(data_bottoms) == 1, "a loss layer reads one score blob and the labels")
            nd.layers.append(nets.softmax_loss().read_from(source(data_bottoms[0])))
            nd.names.append(name)
            done_loss = True
            continue
        if typ == "SPLIT":
            # the reference inserts splits itself; an explicit one only gives the blob more names
            need(len(bottoms) == 1 and tops, "a Split layer has one bottom and at least one top")
            for t in tops:
                writer[t] = source(bottoms[0])
            continue
        if typ == "CONCAT":
            need(2 <= len(bottoms) <= nets.MAX_BOTTOMS and len(tops) == 1,
                 "Concat takes 2..%d bottoms and one top" % nets.MAX_BOTTOMS)
            c = l.msg("concat_param")
            need(int(c.get("axis", c.get("concat_dim", 1))) == 1, "only concatenation along the channel axis is on this path")
            nd.layers.append(nets.concat(*[source(b) for b in bottoms]))
            nd.names.append(name)
            writer[tops[0]] = len(nd.layers) - 1
            continue
        if len(bottoms) != 1 or len(tops) != 1:
            raise PrototxtError("layer %r (%s): one bottom and one top expected" % (name, l.get("type")))
        if tops[0] != name and tops[0] != bottoms[0]:
            raise PrototxtError("layer %r: the top must be the layer's name or its bottom (src/DeepNet.h:847-850)"
                                % name)
        in_place = tops[0] == bottoms[0]
        lr, decay = _multipliers(l)
        if typ == "CONVOLUTION":
            c = l.msg("convolution_param")
            if not c.has("num_output") or not c.has("kernel_size"):
                raise PrototxtError("layer %r: num_output and kernel_size are required" % name)
            g = int(c.get("group", 1))
            need(int(c.get("num_output")) >= 1 and int(c.get("kernel_size")) >= 1, "num_output and kernel_size must be >= 1")
            need(int(c.get("stride", 1)) >= 1 and int(c.get("pad", 0)) >= 0 and g >= 1, "stride and group must be >= 1, pad >= 0")
            spec = nets.conv(int(c.get("num_output")), int(c.get("kernel_size")), stride=int(c.get("stride", 1)),
                             pad=int(c.get("pad", 0)), group=g if groups == "honor" else 1,
                             bias_term=int(bool(c.get("bias_term", True))), lr_mult=lr, decay_mult=decay)
            spec.weight_filler = _filler(c.msg("weight_filler"), "weight_filler", name)
            spec.bias_filler = _filler(c.msg("bias_filler"), "bias_filler", name)
        elif typ == "INNERPRODUCT":
            c = l.msg("inner_product_param")
            if not c.has("num_output"):
                raise PrototxtError("layer %r: num_output is required" % name)
            need(int(c.get("num_output")) >= 1, "num_output must be >= 1")
            spec = nets.fc(int(c.get("num_output")), bias_term=int(bool(c.get("bias_term", True))),
                           lr_mult=lr, decay_mult=decay)
            spec.weight_filler = _filler(c.msg("weight_filler"), "weight_filler", name)
            spec.bias_filler = _filler(c.msg("bias_filler"), "bias_filler", name)
        elif typ == "POOLING":
            c = l.msg("pooling_param")
            if str(c.get("pool", "MAX")) not in ("MAX", "0"):
                raise PrototxtError("layer %r: only MAX pooling is on this path" % name)
            if int(c.get("pad", 0)) != 0:
                raise PrototxtError("layer %r: padded pooling is not supported (src/DeepNet.h:1374-1376)" % name)
            if not c.has("kernel_size"):
                raise PrototxtError("layer %r: kernel_size is required" % name)
            need(int(c.get("kernel_size")) >= 1 and int(c.get("stride", 1)) >= 1, "kernel_size and stride must be >= 1")
            spec = nets.maxpool(int(c.get("kernel_size")), int(c.get("stride", 1)))
        elif typ == "RELU":
            spec = nets.relu()
        elif typ == "LRN":
            c = l.msg("lrn_param")
            if str(c.get("norm_region", "ACROSS_CHANNELS")) not in ("ACROSS_CHANNELS", "0"):
                raise PrototxtError("layer %r: only ACROSS_CHANNELS normalisation is on this path" % name)
            need(int(c.get("local_size", 5)) >= 1 and int(c.get("local_size", 5)) % 2 == 1, "local_size must be odd and >= 1")
            spec = nets.lrn(int(c.get("local_size", 5)), float(c.get("alpha", 1.0)), float(c.get("beta", 0.75)))
        elif typ == "DROPOUT":
            ratio = float(l.msg("dropout_param").get("dropout_ratio", 0.5))
            need(0.0 <= ratio < 1.0, "dropout_ratio must be in [0, 1)")
            spec = nets.dropout(ratio)
        else:
            raise PrototxtError("layer %r: type %r is not supported by this front end" % (name, l.get("type")))
        if in_place and typ not in ("RELU", "DROPOUT"):
            raise PrototxtError("layer %r (%s) cannot run in place" % (name, l.get("type")))
        if not in_place and typ in ("RELU", "DROPOUT"):
            raise PrototxtError("layer %r (%s) must run in place (top == bottom) on this path" % (name, l.get("type")))
        nd.layers.append(spec.read_from(source(bottoms[0])))
        nd.names.append(name)
        writer[tops[0]] = len(nd.layers) - 1
    if not done_loss:
        raise PrototxtError("the network has no SoftmaxWithLoss layer")
    return nd


def load_solver(solver_path, root=None, phase="TRAIN", groups="honor"):
    """Reads a solver file and the network file its `net:` names (paths in the reference's files are
    relative to the directory `caffe-ct` is started from; pass it as `root`).
    Returns (cct_solver_param, control dict, NetworkDef)."""
    sp, control = solver_from_prototxt(parse_file(solver_path))
    if not control["net"]:
        raise PrototxtError("%s: the solver names no `net`" % solver_path)
    net_path = control["net"]
    if not os.path.isabs(net_path):
        net_path = os.path.join(root or os.getcwd(), net_path)
    return sp, control, network_from_prototxt(parse_file(net_path), phase=phase, groups=groups)
