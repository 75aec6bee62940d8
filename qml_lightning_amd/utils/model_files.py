"""Reading TorchScript model files (what ``torch.jit.script(model).save(file)`` writes,
qml_lightning/models/hadamard_features.py:253-255, random_features.py:233-235) WITHOUT
unpickling them and without their operators being registered.

A model file is a zip archive: ``<name>/data.pkl`` (the attribute tree as a pickle program),
``<name>/data/<key>`` (raw little-endian storages), ``<name>/code/**.py`` (TorchScript
source) and ``<name>/version``.  ``torch.jit.load`` needs the operator libraries, a GPU (the
storages of a trained model are tagged ``cuda:0``) and executes the archive's code;
nothing of that is needed to get the weights out.  Here the pickle program is *walked*
with ``pickletools.genops``: a small stack machine over a whitelist of opcodes that builds
plain Python containers and inert placeholder nodes for GLOBAL / REDUCE / NEWOBJ / BUILD /
BINPERSID.  Nothing named in the file is imported, looked up or called; an opcode outside
the whitelist, or a callable other than the four that TorchScript archives use for tensors,
devices and ordered dictionaries, is an error.

    tree = read_attribute_tree("model_sorf.pt")      # nested dict of numpy arrays / scalars
    ops  = called_operators("model_sorf.pt")         # {"qml_lightning_sorf::get_cos_features": [4], ...}
"""
import pickletools
import re
import zipfile

import numpy as np

_STORAGE_DTYPES = {
    "DoubleStorage": "<f8", "FloatStorage": "<f4", "HalfStorage": "<f2", "LongStorage": "<i8",
    "IntStorage": "<i4", "ShortStorage": "<i2", "CharStorage": "i1", "ByteStorage": "u1", "BoolStorage": "?",
}


class _Global:
    """A (module, name) pair named by a GLOBAL opcode: a label, never resolved."""
    __slots__ = ("module", "name")

    def __init__(self, module, name):
        self.module, self.name = module, name

    def __repr__(self):
        return "<%s.%s>" % (self.module, self.name)


class _Call:
    __slots__ = ("func", "args")

    def __init__(self, func, args):
        self.func, self.args = func, args


class _Object:
    __slots__ = ("cls", "args", "state")

    def __init__(self, cls, args):
        self.cls, self.args, self.state = cls, args, None


class _PersId:
    __slots__ = ("pid",)

    def __init__(self, pid):
        self.pid = pid


class _Mark:
    pass


def _walk_pickle(data):
    """Run the pickle program symbolically; returns the object left by STOP."""
    stack, memo = [], {}

    def pop_mark():
        items = []
        while True:
            v = stack.pop()
            if isinstance(v, _Mark):
                break
            items.append(v)
        items.reverse()
        return items

    for op, arg, pos in pickletools.genops(data):
        n = op.name
        if n in ("PROTO", "FRAME"):
            continue
        elif n == "STOP":
            return stack.pop()
        elif n in ("GLOBAL",):
            module, name = arg.split(" ", 1)
            stack.append(_Global(module, name))
        elif n == "STACK_GLOBAL":
            name, module = stack.pop(), stack.pop()
            stack.append(_Global(module, name))
        elif n in ("BINPUT", "LONG_BINPUT", "PUT"):
            memo[arg] = stack[-1]
        elif n == "MEMOIZE":
            memo[len(memo)] = stack[-1]
        elif n in ("BINGET", "LONG_BINGET", "GET"):
            stack.append(memo[arg])
        elif n == "MARK":
            stack.append(_Mark())
        elif n in ("BINUNICODE", "SHORT_BINUNICODE", "BINUNICODE8", "UNICODE", "BININT", "BININT1", "BININT2", "LONG1",
                   "LONG4", "INT", "LONG", "BINFLOAT", "FLOAT", "BINBYTES", "SHORT_BINBYTES", "BINSTRING",
                   "SHORT_BINSTRING"):
            stack.append(arg)
        elif n == "NEWTRUE":
            stack.append(True)
        elif n == "NEWFALSE":
            stack.append(False)
        elif n == "NONE":
            stack.append(None)
        elif n == "EMPTY_TUPLE":
            stack.append(())
        elif n == "TUPLE1":
            stack[-1:] = [(stack[-1],)]
        elif n == "TUPLE2":
            stack[-2:] = [(stack[-2], stack[-1])]
        elif n == "TUPLE3":
            stack[-3:] = [(stack[-3], stack[-2], stack[-1])]
        elif n == "TUPLE":
            stack.append(tuple(pop_mark()))
        elif n == "EMPTY_LIST":
            stack.append([])
        elif n == "LIST":
            stack.append(pop_mark())
        elif n == "APPEND":
            v = stack.pop()
            stack[-1].append(v)
        elif n == "APPENDS":
            items = pop_mark()
            stack[-1].extend(items)
        elif n == "EMPTY_DICT":
            stack.append({})
        elif n == "DICT":
            items = pop_mark()
            stack.append(dict(zip(items[0::2], items[1::2])))
        elif n == "SETITEM":
            v, k = stack.pop(), stack.pop()
            _setitem(stack[-1], k, v)
        elif n == "SETITEMS":
            items = pop_mark()
            for k, v in zip(items[0::2], items[1::2]):
                _setitem(stack[-1], k, v)
        elif n == "BINPERSID":
            stack.append(_PersId(stack.pop()))
        elif n == "REDUCE":
            args, func = stack.pop(), stack.pop()
            stack.append(_Call(func, args))
        elif n == "NEWOBJ":
            args, cls = stack.pop(), stack.pop()
            stack.append(_Object(cls, args))
        elif n == "BUILD":
            state = stack.pop()
            target = stack[-1]
            if not isinstance(target, _Object):
                raise ValueError("model file: BUILD on something that is not an object (offset %d)" % pos)
            target.state = state
        else:
            raise ValueError("model file: pickle opcode %s (offset %d) is not one a TorchScript archive uses" % (n, pos))
    raise ValueError("model file: pickle program without STOP")


def _setitem(target, k, v):
    if isinstance(target, dict):
        target[k] = v
    elif isinstance(target, _Call) and isinstance(target.func, _Global) and target.func.name == "OrderedDict":
        if not isinstance(target.args, dict):
            target.args = {}
        target.args[k] = v
    else:
        raise ValueError("model file: item assignment on an unexpected object")


class _Archive:
    def __init__(self, path):
        self.zip = zipfile.ZipFile(path)
        names = self.zip.namelist()
        roots = {n.split("/", 1)[0] for n in names if n.endswith("/data.pkl") and n.count("/") == 1}
        if len(roots) != 1:
            raise ValueError("%s: not a TorchScript archive (no single <name>/data.pkl)" % path)
        self.root = roots.pop()
        self.names = names
        self._storages = {}

    def read(self, rel):
        return self.zip.read(self.root + "/" + rel)

    def storage(self, key, dtype):
        k = (key, dtype)
        if k not in self._storages:
            self._storages[k] = np.frombuffer(self.read("data/%s" % key), dtype=dtype)
        return self._storages[k]


def _tensor(ar, call):
    """numpy array of a `torch._utils._rebuild_tensor_v2(storage, offset, size, stride, ...)` node."""
    pers, offset, size, stride = call.args[0], call.args[1], call.args[2], call.args[3]
    if not isinstance(pers, _PersId) or pers.pid[0] != "storage":
        raise ValueError("model file: tensor without a storage record")
    _, stype, key, location, numel = pers.pid[:5]
    if not isinstance(stype, _Global) or stype.name not in _STORAGE_DTYPES:
        raise ValueError("model file: storage class %r is not known" % (stype,))
    dtype = _STORAGE_DTYPES[stype.name]
    flat = ar.storage(key, dtype)
    if flat.shape[0] < numel:
        raise ValueError("model file: storage %s holds %d elements, %d are recorded" % (key, flat.shape[0], numel))
    size, stride = tuple(int(s) for s in size), tuple(int(s) for s in stride)
    span = offset + 1 + sum((s - 1) * st for s, st in zip(size, stride)) if all(s > 0 for s in size) else offset
    if span > flat.shape[0]:
        raise ValueError("model file: tensor reaches past the end of storage %s" % key)
    itemsize = flat.dtype.itemsize
    view = np.lib.stride_tricks.as_strided(flat[offset:], shape=size, strides=tuple(st * itemsize for st in stride),
                                           writeable=False)
    return np.array(view)      # an owned, contiguous copy


def _resolve(ar, node):
    if isinstance(node, _Object):
        out = {"__class__": "%s.%s" % (node.cls.module, node.cls.name)}
        state = node.state if node.state is not None else {}
        for k, v in state.items():
            out[k] = _resolve(ar, v)
        return out
    if isinstance(node, _Call):
        f = node.func
        if isinstance(f, _Global) and (f.module, f.name) == ("torch._utils", "_rebuild_tensor_v2"):
            return _tensor(ar, node)
        if isinstance(f, _Global) and (f.module, f.name) == ("torch", "device"):
            return "device(%s)" % ", ".join(str(a) for a in node.args)
        if isinstance(f, _Global) and f.name == "OrderedDict":
            d = node.args if isinstance(node.args, dict) else {}
            return {k: _resolve(ar, v) for k, v in d.items()}
        if isinstance(f, _Global) and (f.module, f.name) == ("torch._utils", "_rebuild_parameter"):
            return _resolve(ar, node.args[0])
        raise ValueError("model file: call of %r is not one a TorchScript archive uses" % (f,))
    if isinstance(node, dict):
        return {k: _resolve(ar, v) for k, v in node.items()}
    if isinstance(node, (list, tuple)):
        return type(node)(_resolve(ar, v) for v in node)
    if isinstance(node, (_Global, _PersId)):
        raise ValueError("model file: unexpected bare %s in the attribute tree" % type(node).__name__)
    return node


def read_attribute_tree(path):
    """The module's attributes as a nested dict: tensors as numpy arrays (dtype and shape as
    saved), Python scalars as they are, sub-modules as nested dicts; every module dict carries
    its TorchScript class name under ``"__class__"``."""
    ar = _Archive(path)
    return _resolve(ar, _walk_pickle(ar.read("data.pkl")))


def archive_version(path):
    return int(_Archive(path).read("version").decode().strip())


def archive_code(path):
    """{relative file name: TorchScript source text} of the archive's ``code/`` tree."""
    ar = _Archive(path)
    pre = ar.root + "/code/"
    return {n[len(pre):]: ar.zip.read(n).decode() for n in ar.names if n.startswith(pre) and n.endswith(".py")}


_OP_CALL = re.compile(r"\bops\.(\w+)\.(\w+)\(")


def _split_args(text, start):
    """Argument strings of the call whose opening parenthesis is at text[start]."""
    depth, args, cur, i, quote = 0, [], [], start, None
    while i < len(text):
        c = text[i]
        if quote:
            cur.append(c)
            if c == "\\":
                cur.append(text[i + 1])
                i += 1
            elif c == quote:
                quote = None
        elif c in "\"'":
            quote = c
            cur.append(c)
        elif c in "([{":
            depth += 1
            if depth > 1:
                cur.append(c)
        elif c in ")]}":
            depth -= 1
            if depth == 0:
                s = "".join(cur).strip()
                if s:
                    args.append(s)
                return args
            cur.append(c)
        elif c == "," and depth == 1:
            args.append("".join(cur).strip())
            cur = []
        else:
            cur.append(c)
        i += 1
    raise ValueError("unbalanced call in TorchScript source")


def called_operators(path, namespaces=("qml_lightning_fchl", "qml_lightning_sorf")):
    """Custom operators the archive's code calls: {"namespace::name": [argument lists]}, each
    argument list as the source strings of that call's arguments (a keyword argument shows as
    ``"name=value"``).  Built-in namespaces (``ops.prim`` ...) are left out."""
    found = {}
    for _, src in sorted(archive_code(path).items()):
        for m in _OP_CALL.finditer(src):
            if m.group(1) not in namespaces:
                continue
            found.setdefault("%s::%s" % (m.group(1), m.group(2)), []).append(_split_args(src, m.end() - 1))
    return found


# The operators of the reference's two TorchScript libraries with their argument counts: schemas are
# inferred from plain C++ functions taking at::Tensor, so every argument is a positional Tensor
# (torchscript/FCHL19.cpp:318-333, torchscript/SORF.cpp:138-150).
REFERENCE_OPERATORS = {
    "qml_lightning_fchl::fchl_forwards": 16,
    "qml_lightning_fchl::get_fchl_and_derivative": 17,
    "qml_lightning_fchl::get_element_types": 4,
    "qml_lightning_fchl::get_neighbour_list": 6,
    "qml_lightning_fchl::get_num_neighbours": 5,
    "qml_lightning_sorf::get_SORF_coefficients": 4,
    "qml_lightning_sorf::get_cos_features": 4,
}


def check_reference_loadable(path):
    """Raise ValueError unless the archive calls only operators the reference registers, each with
    the reference's positional argument count and no keyword arguments: the condition for a host
    that has the reference's operator libraries (and not this package's extra operators) to load
    and run the file.  Returns the {operator: number of call sites} it found."""
    calls = called_operators(path)
    for name, sites in calls.items():
        if name not in REFERENCE_OPERATORS:
            raise ValueError("%s calls %s, which the reference's operator libraries do not register" % (path, name))
        for args in sites:
            if len(args) != REFERENCE_OPERATORS[name]:
                raise ValueError("%s calls %s with %d arguments, the reference's schema has %d"
                                 % (path, name, len(args), REFERENCE_OPERATORS[name]))
            if any(re.match(r"^\w+\s*=[^=]", a) for a in args):
                raise ValueError("%s calls %s with a keyword argument" % (path, name))
    return {k: len(v) for k, v in calls.items()}
