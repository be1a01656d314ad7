"""Reader for deepnet's text-format configuration files (model / operation .pbtxt, the files
deepnet/util.py:55-93 reads with protobuf's text_format.Merge) without generated protobuf
classes: the text is parsed into a tree of ``Message`` objects that keep which fields were
written, so that "merge the fields that are set" (the MergeFrom of deepnet/neuralnet.py:78-93)
can be done on them.  Only the grammar is known here, not the schema: every field holds the
list of values written for it, ``get`` returns the last one (what a non-repeated field ends
up with), ``all`` the list (a repeated field).  Enum values stay as their names.
"""
import re

_TOKEN = re.compile(r"""
    \s+ | \#[^\n]*                                   # blanks and comments
  | (?P<str>"(?:[^"\\\n]|\\.)*" | '(?:[^'\\\n]|\\.)*')
  | (?P<num>[-+]?(?:\d+\.?\d*(?:[eE][-+]?\d+)?|\.\d+(?:[eE][-+]?\d+)?|inf|nan)f?(?![\w.]))
  | (?P<name>[A-Za-z_][\w.]*)
  | (?P<punct>[{}<>:;,\[\]])
""", re.VERBOSE)

_ESCAPES = {'n': '\n', 't': '\t', 'r': '\r', '\\': '\\', '"': '"', "'": "'", '0': '\0'}


class ParseError(ValueError):
    pass


class Enum(str):
    """An enum value, kept by name: compares like the string, written back without quotes."""


class Message(object):
    """Fields in the order written.  ``msg.get('dimensions')``, ``msg.all('shape')``,
    ``'hyperparams' in msg``; attribute access is ``get`` and raises for a field not written."""

    def __init__(self, fields=None):
        self._fields = list(fields or [])

    def add(self, name, value):
        self._fields.append((name, value))

    def all(self, name):
        return [v for n, v in self._fields if n == name]

    def get(self, name, default=None):
        for n, v in reversed(self._fields):
            if n == name:
                return v
        return default

    def set(self, name, *values):
        """Replace whatever was written for ``name`` by ``values`` (at the position of the
        first occurrence, or at the end)."""
        at = next((i for i, (n, _) in enumerate(self._fields) if n == name), len(self._fields))
        kept = [(n, v) for n, v in self._fields if n != name]
        at = min(at, len(kept))
        self._fields = kept[:at] + [(name, v) for v in values] + kept[at:]

    def names(self):
        seen = []
        for n, _ in self._fields:
            if n not in seen:
                seen.append(n)
        return seen

    def scalars(self):
        """{name: last value} of the fields that are not sub-messages."""
        return {n: v for n, v in self._fields if not isinstance(v, Message)}

    def __contains__(self, name):
        return any(n == name for n, _ in self._fields)

    def __getattr__(self, name):
        if name.startswith('_'):
            raise AttributeError(name)
        for n, v in reversed(self._fields):
            if n == name:
                return v
        raise AttributeError('field %r was not written' % name)

    def __eq__(self, other):
        return isinstance(other, Message) and self._fields == other._fields

    def __repr__(self):
        return 'Message(%r)' % (self._fields,)


def _tokens(text):
    pos, line = 0, 1
    while pos < len(text):
        m = _TOKEN.match(text, pos)
        if not m:
            raise ParseError('line %d: cannot read %r' % (line, text[pos:pos + 20]))
        line += text.count('\n', pos, m.end())
        pos = m.end()
        if m.lastgroup:
            yield m.lastgroup, m.group(m.lastgroup), line
    yield 'end', '', line


def _unquote(tok):
    body, out, i = tok[1:-1], [], 0
    while i < len(body):
        c = body[i]
        if c == '\\':
            i += 1
            e = body[i]
            if e == 'x':
                out.append(chr(int(body[i + 1:i + 3], 16)))
                i += 2
            elif e in '01234567':                     # one to three octal digits
                j = i + 1
                while j < len(body) and j < i + 3 and body[j] in '01234567':
                    j += 1
                out.append(chr(int(body[i:j], 8) & 0xff))
                i = j - 1
            else:
                out.append(_ESCAPES.get(e, e))
        else:
            out.append(c)
        i += 1
    return ''.join(out)


def _number(tok):
    t = tok[:-1] if tok.endswith('f') and not tok.endswith('inf') else tok
    try:
        return int(t)
    except ValueError:
        return float(t)


class _Parser(object):
    def __init__(self, text):
        self.toks = list(_tokens(text))
        self.i = 0

    def peek(self):
        return self.toks[self.i]

    def take(self):
        t = self.toks[self.i]
        self.i += 1
        return t

    def fail(self, what):
        kind, val, line = self.peek()
        raise ParseError('line %d: %s, found %r' % (line, what, val or kind))

    def message(self, closer):
        msg = Message()
        while True:
            kind, val, _ = self.peek()
            if kind == 'punct' and val in ',;':
                self.take()
                continue
            if closer is None and kind == 'end':
                return msg
            if closer is not None and kind == 'punct' and val == closer:
                self.take()
                return msg
            if kind != 'name':
                self.fail('expected a field name')
            name = self.take()[1]
            kind, val, _ = self.peek()
            colon = kind == 'punct' and val == ':'
            if colon:
                self.take()
                kind, val, _ = self.peek()
            if kind == 'punct' and val in '{<':
                self.take()
                msg.add(name, self.message('}' if val == '{' else '>'))
            elif not colon:
                self.fail("expected ':' or '{' after %s" % name)
            elif kind == 'punct' and val == '[':
                self.take()
                while True:
                    kind, val, _ = self.peek()
                    if kind == 'punct' and val == ']':
                        self.take()
                        break
                    if kind == 'punct' and val == ',':
                        self.take()
                        continue
                    msg.add(name, self.scalar())
            else:
                msg.add(name, self.scalar())

    def scalar(self):
        kind, val, _ = self.peek()
        if kind == 'str':
            parts = []
            while self.peek()[0] == 'str':           # adjacent strings concatenate
                parts.append(_unquote(self.take()[1]))
            return ''.join(parts)
        if kind == 'num':
            return _number(self.take()[1])
        if kind == 'name':
            self.take()
            if val in ('true', 'True', 't'):
                return True
            if val in ('false', 'False', 'f'):
                return False
            if val in ('inf', 'infinity', 'nan'):
                return float(val[:3])
            return Enum(val)                          # an enum value, by name
        self.fail('expected a value')


def parse(text):
    """The top-level message of a text-format file."""
    return _Parser(text).message(None)


def merged(base, over):
    """``base`` with the fields written in ``over`` on top: non-repeated semantics, scalar
    fields replaced, sub-messages merged recursively (protobuf's MergeFrom for the messages
    deepnet merges, which hold no repeated fields)."""
    out = Message()
    for name in list(base.names() if base else []) + [n for n in (over.names() if over else []) if not base or n not in base]:
        b = base.get(name) if base and name in base else None
        o = over.get(name) if over and name in over else None
        if isinstance(b, Message) or isinstance(o, Message):
            out.add(name, merged(b if isinstance(b, Message) else None, o if isinstance(o, Message) else None))
        else:
            out.add(name, o if o is not None else b)
    return out


def _quote(raw):
    """A bytes or str value as a double-quoted literal in printable ASCII (octal escapes, as
    protobuf's text_format writes bytes fields)."""
    # a parsed bytes field is a str with one character per byte: those go back out as the bytes
    # they stand for (latin-1); only text with characters beyond 0xFF is written as UTF-8
    if isinstance(raw, bytes):
        data = raw
    else:
        try:
            data = raw.encode('latin-1')
        except UnicodeEncodeError:
            data = raw.encode('utf-8')
    out = []
    for b in data:
        c = chr(b)
        if c in '"\\':
            out.append('\\' + c)
        elif c == '\n':
            out.append('\\n')
        elif 32 <= b < 127:
            out.append(c)
        else:
            out.append('\\%03o' % b)
    return '"' + ''.join(out) + '"'


def dumps(msg, indent=0):
    """The text form of a message tree; ``parse(dumps(m)) == m`` for trees made of Message, Enum,
    bool, int, float and str values (bytes values come back as str with one character per byte)."""
    pad, lines = '  ' * indent, []
    for name, v in msg._fields:
        if isinstance(v, Message):
            lines.append('%s%s {\n%s%s}\n' % (pad, name, dumps(v, indent + 1), pad))
        elif isinstance(v, bool):
            lines.append('%s%s: %s\n' % (pad, name, 'true' if v else 'false'))
        elif isinstance(v, Enum):
            lines.append('%s%s: %s\n' % (pad, name, v))
        elif isinstance(v, (bytes, str)):
            lines.append('%s%s: %s\n' % (pad, name, _quote(v)))
        else:
            lines.append('%s%s: %r\n' % (pad, name, v))
    return ''.join(lines)
