"""Chat templates: `ChatTemplate` of the reference's chat front end
(crates/wgml-chat/src/chat_template.rs:5-40) and the `Prompt` it renders
(crates/wgml-chat/src/prompt.rs:15-108).

The reference hands the template text (GGUF key `tokenizer.chat_template`, or the Llama-2
default of models/llama2/tokenizer.rs:19-21) to the minijinja crate with `trim_blocks` on and
the globals `bos_token`, `eos_token`, `add_generation_prompt = true`, and `messages` as a list
of {role, content} maps.  No template engine is importable here, so this module carries a small
interpreter of the Jinja subset chat templates are written in:

  statements   if / elif / else / endif, for x in seq / endfor (with `loop.index0`, `index`,
               `first`, `last`, `length`), set name = expr, set ns.attr = expr, comments
  whitespace   `{%-`, `-%}`, `{{-`, `-}}` strip the neighbouring text; with trim_blocks the first
               newline after a block tag is dropped (not after `{{ }}`), as Jinja defines it
  expressions  strings, integers, true / false / none, names, `a.b`, `a[b]`, `a[i:j]`, calls,
               `+ - * // % ~`, comparisons, `in` / `not in`, `and` / `or` / `not`,
               `x if c else y`, filters (`trim`, `last`, `first`, `length`, `split`, `upper`,
               `lower`, `default`, `join`, `tojson`), tests (`defined`, `none`, `string`,
               `true`, `false`), string methods (`strip`, `split`, `startswith`, `endswith`,
               `upper`, `lower`, `replace`), `raise_exception(msg)`, `namespace(...)`
  precedence   as in Jinja: a filter binds tighter than an arithmetic operator, so
               `a + b | trim` is `a + (b | trim)`

An undefined name renders as the empty string and is false in a condition (the engine's
default, lenient behaviour).
"""
from __future__ import annotations

import json
import re
from typing import Any, Dict, List, Optional, Sequence

__all__ = ["ChatTemplate", "Prompt", "TemplateError", "LLAMA2_CHAT_TEMPLATE"]

# The reference's default template for Llama-family models (llama-2-chat.jinja, credited there to
# github.com/chujiezheng/chat_templates, MIT licence): GGUF files normally carry their own under
# `tokenizer.chat_template`; this is what `ChatTemplate::from_gguf` falls back to.
LLAMA2_CHAT_TEMPLATE = (
    "{% if messages[0]['role'] == 'system' %}\n"
    "    {% set system_message = '<<SYS>>\\n' + messages[0]['content'] | trim + '\\n<</SYS>>\\n\\n' %}\n"
    "    {% set messages = messages[1:] %}\n"
    "{% else %}\n"
    "    {% set system_message = '' %}\n"
    "{% endif %}\n"
    "\n"
    "{% for message in messages %}\n"
    "    {% if (message['role'] == 'user') != (loop.index0 % 2 == 0) %}\n"
    "        {{ raise_exception('Conversation roles must alternate user/assistant/user/assistant/...') }}\n"
    "    {% endif %}\n"
    "\n"
    "    {% if loop.index0 == 0 %}\n"
    "        {% set content = system_message + message['content'] %}\n"
    "    {% else %}\n"
    "        {% set content = message['content'] %}\n"
    "    {% endif %}\n"
    "\n"
    "    {% if message['role'] == 'user' %}\n"
    "        {{ bos_token + '[INST] ' + content | trim + ' [/INST]' }}\n"
    "    {% elif message['role'] == 'assistant' %}\n"
    "        {{ ' ' + content | trim + ' ' + eos_token }}\n"
    "    {% endif %}\n"
    "{% endfor %}"
)


class TemplateError(ValueError):
    """A template that does not parse, or `raise_exception(...)` called by one."""


class _Undefined:
    def __bool__(self):
        return False

    def __str__(self):
        return ""

    def __iter__(self):
        return iter(())

    def __len__(self):
        return 0

    def __eq__(self, other):
        return isinstance(other, _Undefined)

    def __hash__(self):
        return 0


UNDEFINED = _Undefined()


class _Namespace:
    def __init__(self, **kw):
        self.__dict__.update(kw)


# ---- lexer ------------------------------------------------------------------------------------
_TAG = re.compile(r"\{\{-?|\{%-?|\{#-?")
_EXPR_TOKEN = re.compile(
    r"\s*(?:(?P<num>\d+(?:\.\d+)?)|(?P<name>[A-Za-z_][A-Za-z0-9_]*)|(?P<str>'(?:\\.|[^'\\])*'|\"(?:\\.|[^\"\\])*\")"
    r"|(?P<op>==|!=|<=|>=|//|\*\*|[-+*/%~<>()\[\]{}.,:|=]))")


def _unescape(body: str) -> str:
    out, i = [], 0
    simple = {"n": "\n", "t": "\t", "r": "\r", "\\": "\\", "'": "'", '"': '"', "0": "\0"}
    while i < len(body):
        c = body[i]
        if c == "\\" and i + 1 < len(body):
            out.append(simple.get(body[i + 1], "\\" + body[i + 1]))
            i += 2
        else:
            out.append(c)
            i += 1
    return "".join(out)


def _split_source(src: str, trim_blocks: bool):
    """-> list of ('text', s) | ('var', expr) | ('block', stmt)."""
    out: List[tuple] = []
    pos = 0
    strip_next = False    # a `-%}` / `-}}` before: strip leading whitespace of the next text
    after_block = False   # a block tag before: trim_blocks drops one leading newline
    while True:
        m = _TAG.search(src, pos)
        text = src[pos:m.start()] if m else src[pos:]
        if strip_next:
            text = text.lstrip()
        elif after_block and trim_blocks:
            if text.startswith("\r\n"):
                text = text[2:]
            elif text.startswith("\n"):
                text = text[1:]
        if m and m.group().endswith("-"):
            text = text.rstrip()
        if text:
            out.append(("text", text))
        if not m:
            break
        kind = m.group()[:2]
        close = {"{{": "}}", "{%": "%}", "{#": "#}"}[kind]
        end = src.find(close, m.end())
        if end < 0:
            raise TemplateError(f"unclosed {kind} at offset {m.start()}")
        body = src[m.end():end]
        strip_next = body.endswith("-")
        if strip_next:
            body = body[:-1]
        pos = end + 2
        after_block = kind != "{{"
        if kind == "{{":
            out.append(("var", body.strip()))
        elif kind == "{%":
            out.append(("block", body.strip()))
    return out


# ---- expressions: tokens -> closures over an environment -----------------------------------------
class _Expr:
    def __init__(self, text: str):
        self.toks: List[tuple] = []
        pos = 0
        text = text.strip()
        while pos < len(text):
            m = _EXPR_TOKEN.match(text, pos)
            if not m or m.end() == pos:
                if text[pos:].strip() == "":
                    break
                raise TemplateError(f"cannot read expression at {text[pos:pos + 20]!r}")
            pos = m.end()
            for k in ("num", "name", "str", "op"):
                if m.group(k) is not None:
                    self.toks.append((k, m.group(k)))
                    break
        self.i = 0

    def peek(self, value=None):
        if self.i >= len(self.toks):
            return None
        k, v = self.toks[self.i]
        if value is None:
            return v
        return v if (v == value and k in ("op", "name")) else None

    def take(self, value=None):
        v = self.peek(value)
        if v is None:
            raise TemplateError(f"expected {value!r} in expression, got {self.peek()!r}")
        self.i += 1
        return v

    def done(self):
        return self.i >= len(self.toks)

    # grammar, loosest first
    def parse(self):
        return self.ternary()

    def ternary(self):
        a = self.or_()
        if self.peek("if"):
            self.take()
            c = self.or_()
            b = (lambda env: UNDEFINED)
            if self.peek("else"):
                self.take()
                b = self.ternary()
            return lambda env, a=a, b=b, c=c: a(env) if _truth(c(env)) else b(env)
        return a

    def or_(self):
        a = self.and_()
        while self.peek("or"):
            self.take()
            b = self.and_()
            a = (lambda env, a=a, b=b: (lambda x: x if _truth(x) else b(env))(a(env)))
        return a

    def and_(self):
        a = self.not_()
        while self.peek("and"):
            self.take()
            b = self.not_()
            a = (lambda env, a=a, b=b: (lambda x: b(env) if _truth(x) else x)(a(env)))
        return a

    def not_(self):
        if self.peek("not"):
            self.take()
            a = self.not_()
            return lambda env, a=a: not _truth(a(env))
        return self.compare()

    def compare(self):
        a = self.additive()
        while True:
            op = self.peek()
            if op in ("==", "!=", "<", ">", "<=", ">="):
                self.take()
                b = self.additive()
                a = _binary(op, a, b)
            elif op == "in":
                self.take()
                b = self.additive()
                a = (lambda env, a=a, b=b: _contains(b(env), a(env)))
            elif op == "not" and self.i + 1 < len(self.toks) and self.toks[self.i + 1][1] == "in":
                self.take()
                self.take()
                b = self.additive()
                a = (lambda env, a=a, b=b: not _contains(b(env), a(env)))
            elif op == "is":
                self.take()
                neg = bool(self.peek("not"))
                if neg:
                    self.take()
                name = self.take()
                a = _test(name, a, neg)
            else:
                return a

    def additive(self):
        a = self.term()
        while self.peek() in ("+", "-", "~"):
            op = self.take()
            b = self.term()
            a = _binary(op, a, b)
        return a

    def term(self):
        a = self.unary()
        while self.peek() in ("*", "/", "//", "%"):
            op = self.take()
            b = self.unary()
            a = _binary(op, a, b)
        return a

    def unary(self):
        if self.peek("-"):
            self.take()
            a = self.unary()
            return lambda env, a=a: -a(env)
        return self.filtered()

    def filtered(self):
        a = self.postfix()
        while self.peek("|"):
            self.take()
            name = self.take()
            args = self.call_args() if self.peek("(") else []
            a = _filter(name, a, args)
        return a

    def call_args(self):
        self.take("(")
        args, kwargs = [], {}
        while not self.peek(")"):
            if (self.i + 1 < len(self.toks) and self.toks[self.i][0] == "name"
                    and self.toks[self.i + 1] == ("op", "=")):
                key = self.take()
                self.take("=")
                kwargs[key] = self.parse()
            else:
                args.append(self.parse())
            if self.peek(","):
                self.take()
        self.take(")")
        return args if not kwargs else args + [("kwargs", kwargs)]

    def postfix(self):
        a = self.primary()
        while True:
            if self.peek("."):
                self.take()
                name = self.take()
                if self.peek("("):
                    args = self.call_args()
                    a = _method(name, a, args)
                else:
                    a = (lambda env, a=a, name=name: _attr(a(env), name))
            elif self.peek("["):
                self.take()
                lo = None if self.peek(":") else self.parse()
                if self.peek(":"):
                    self.take()
                    hi = None if self.peek("]") else self.parse()
                    self.take("]")
                    a = (lambda env, a=a, lo=lo, hi=hi: _slice(a(env), lo(env) if lo else None,
                                                               hi(env) if hi else None))
                else:
                    self.take("]")
                    a = (lambda env, a=a, lo=lo: _index(a(env), lo(env)))
            elif self.peek("("):
                args = self.call_args()
                a = (lambda env, a=a, args=args: _call(a(env), args, env))
            else:
                return a

    def primary(self):
        if self.i >= len(self.toks):
            raise TemplateError("expression ends early")
        k, v = self.toks[self.i]
        self.i += 1
        if k == "num":
            val = float(v) if "." in v else int(v)
            return lambda env, val=val: val
        if k == "str":
            val = _unescape(v[1:-1])
            return lambda env, val=val: val
        if k == "name":
            if v in ("true", "True"):
                return lambda env: True
            if v in ("false", "False"):
                return lambda env: False
            if v in ("none", "None"):
                return lambda env: None
            return lambda env, v=v: env.get(v, UNDEFINED)
        if v == "(":
            a = self.parse()
            self.take(")")
            return a
        if v == "[":
            items = []
            while not self.peek("]"):
                items.append(self.parse())
                if self.peek(","):
                    self.take()
            self.take("]")
            return lambda env, items=items: [f(env) for f in items]
        raise TemplateError(f"unexpected {v!r} in expression")


def _truth(v) -> bool:
    return bool(v)


def _contains(container, item) -> bool:
    try:
        return item in container
    except TypeError:
        return False


def _binary(op, a, b):
    def run(env):
        x, y = a(env), b(env)
        if op == "~":
            return _to_str(x) + _to_str(y)
        if op == "+":
            if isinstance(x, str) or isinstance(y, str):
                return _to_str(x) + _to_str(y)
            return x + y
        if op == "==":
            return x == y
        if op == "!=":
            return x != y
        try:
            return {"-": lambda: x - y, "*": lambda: x * y, "/": lambda: x / y, "//": lambda: x // y,
                    "%": lambda: x % y, "<": lambda: x < y, ">": lambda: x > y, "<=": lambda: x <= y,
                    ">=": lambda: x >= y}[op]()
        except TypeError as e:
            raise TemplateError(f"cannot apply {op!r} to {x!r} and {y!r}") from e
    return run


def _test(name, a, neg):
    def run(env):
        v = a(env)
        r = {"defined": lambda: not isinstance(v, _Undefined), "undefined": lambda: isinstance(v, _Undefined),
             "none": lambda: v is None, "string": lambda: isinstance(v, str),
             "true": lambda: v is True, "false": lambda: v is False,
             "iterable": lambda: isinstance(v, (list, tuple, str, dict)),
             "mapping": lambda: isinstance(v, dict), "number": lambda: isinstance(v, (int, float)) and
             not isinstance(v, bool)}.get(name)
        if r is None:
            raise TemplateError(f"unknown test {name!r}")
        return r() != neg
    return run


def _to_str(v) -> str:
    if v is None:
        return "none"
    if v is True:
        return "true"
    if v is False:
        return "false"
    return str(v)


def _eval_args(args, env):
    pos, kw = [], {}
    for a in args:
        if isinstance(a, tuple) and a and a[0] == "kwargs":
            kw = {k: f(env) for k, f in a[1].items()}
        else:
            pos.append(a(env))
    return pos, kw


def _filter(name, a, args):
    def run(env):
        v = a(env)
        pos, kw = _eval_args(args, env)
        if name in ("trim", "strip"):
            return _to_str(v).strip()
        if name == "last":
            return v[-1] if len(v) else UNDEFINED
        if name == "first":
            return v[0] if len(v) else UNDEFINED
        if name in ("length", "count"):
            return len(v)
        if name == "split":
            return _to_str(v).split(*pos)
        if name == "upper":
            return _to_str(v).upper()
        if name == "lower":
            return _to_str(v).lower()
        if name in ("default", "d"):
            return (pos[0] if pos else "") if isinstance(v, _Undefined) else v
        if name == "join":
            return (pos[0] if pos else "").join(_to_str(x) for x in v)
        if name == "tojson":
            return json.dumps(v, ensure_ascii=False)
        if name == "string":
            return _to_str(v)
        if name == "int":
            return int(v)
        if name == "list":
            return list(v)
        raise TemplateError(f"unknown filter {name!r}")
    return run


def _method(name, a, args):
    def run(env):
        v = a(env)
        pos, kw = _eval_args(args, env)
        if isinstance(v, str) and name in ("strip", "lstrip", "rstrip", "split", "startswith", "endswith",
                                           "upper", "lower", "replace", "title"):
            return getattr(v, name)(*pos)
        if isinstance(v, dict) and name in ("get", "items", "keys", "values"):
            r = getattr(v, name)(*pos)
            return list(r) if name != "get" else (UNDEFINED if r is None and len(pos) < 2 else r)
        raise TemplateError(f"no method {name!r} on {type(v).__name__}")
    return run


def _attr(v, name):
    if isinstance(v, dict):
        return v.get(name, UNDEFINED)
    if isinstance(v, _Namespace) or isinstance(v, _Loop):
        return getattr(v, name, UNDEFINED)
    return UNDEFINED


def _index(v, i):
    try:
        return v[i]
    except (KeyError, IndexError, TypeError):
        return UNDEFINED


def _slice(v, lo, hi):
    try:
        return v[lo:hi]
    except TypeError:
        return UNDEFINED


def _call(fn, args, env):
    pos, kw = _eval_args(args, env)
    if callable(fn):
        return fn(*pos, **kw)
    raise TemplateError("call of something that is not a function")


class _Loop:
    def __init__(self, n):
        self.length = n
        self.index0 = 0

    @property
    def index(self):
        return self.index0 + 1

    @property
    def first(self):
        return self.index0 == 0

    @property
    def last(self):
        return self.index0 == self.length - 1

    @property
    def revindex(self):
        return self.length - self.index0

    @property
    def revindex0(self):
        return self.length - self.index0 - 1


# ---- statements -------------------------------------------------------------------------------------
def _parse_nodes(items, i, stop):
    """Parses until a block whose first word is in `stop`; returns (nodes, index of that block)."""
    nodes = []
    while i < len(items):
        kind, body = items[i]
        if kind == "text":
            nodes.append(("text", body))
            i += 1
        elif kind == "var":
            e = _Expr(body)
            f = e.parse()
            if not e.done():
                raise TemplateError(f"trailing input in {{{{ {body} }}}}")
            nodes.append(("var", f))
            i += 1
        else:
            word = body.split(None, 1)[0] if body else ""
            rest = body[len(word):].strip()
            if word in stop:
                return nodes, i
            if word == "if":
                branches, else_nodes = [], None
                cond = _full_expr(rest)
                while True:
                    inner, i = _parse_nodes(items, i + 1, ("elif", "else", "endif"))
                    if i >= len(items):
                        raise TemplateError("if without endif")
                    if cond is not None:
                        branches.append((cond, inner))
                    else:
                        else_nodes = inner
                    w = items[i][1].split(None, 1)[0]
                    if w == "elif":
                        cond = _full_expr(items[i][1][4:].strip())
                    elif w == "else":
                        cond = None
                    else:
                        break
                nodes.append(("if", branches, else_nodes))
                i += 1
            elif word == "for":
                m = re.match(r"([A-Za-z_][A-Za-z0-9_]*(?:\s*,\s*[A-Za-z_][A-Za-z0-9_]*)*)\s+in\s+(.*)$", rest, re.S)
                if not m:
                    raise TemplateError(f"cannot read for statement {body!r}")
                names = [n.strip() for n in m.group(1).split(",")]
                seq = _full_expr(m.group(2))
                inner, i = _parse_nodes(items, i + 1, ("endfor",))
                if i >= len(items):
                    raise TemplateError("for without endfor")
                nodes.append(("for", names, seq, inner))
                i += 1
            elif word == "set":
                m = re.match(r"([A-Za-z_][A-Za-z0-9_]*)(?:\.([A-Za-z_][A-Za-z0-9_]*))?\s*=(?!=)\s*(.*)$", rest, re.S)
                if not m:
                    raise TemplateError(f"cannot read set statement {body!r}")
                nodes.append(("set", m.group(1), m.group(2), _full_expr(m.group(3))))
                i += 1
            else:
                raise TemplateError(f"unknown statement {word!r}")
    if stop:
        return nodes, i
    return nodes, i


def _full_expr(text):
    e = _Expr(text)
    f = e.parse()
    if not e.done():
        raise TemplateError(f"trailing input in expression {text!r}")
    return f


def _render(nodes, env: Dict[str, Any], out: List[str]):
    for n in nodes:
        k = n[0]
        if k == "text":
            out.append(n[1])
        elif k == "var":
            v = n[1](env)
            out.append("" if v is None or isinstance(v, _Undefined) else _to_str(v))
        elif k == "if":
            for cond, inner in n[1]:
                if _truth(cond(env)):
                    _render(inner, env, out)
                    break
            else:
                if n[2] is not None:
                    _render(n[2], env, out)
        elif k == "for":
            seq = n[2](env)
            seq = list(seq.items()) if isinstance(seq, dict) else list(seq)
            loop = _Loop(len(seq))
            # a loop body has its own scope: names it sets do not leak out (Jinja's rule;
            # `namespace` objects exist for what must outlive an iteration)
            for idx, item in enumerate(seq):
                scope = dict(env)
                loop.index0 = idx
                scope["loop"] = loop
                if len(n[1]) == 1:
                    scope[n[1][0]] = item
                else:
                    for name, v in zip(n[1], item):
                        scope[name] = v
                _render(n[3], scope, out)
        elif k == "set":
            val = n[3](env)
            if n[2] is None:
                env[n[1]] = val
            else:
                target = env.get(n[1])
                if not isinstance(target, _Namespace):
                    raise TemplateError(f"{n[1]} is not a namespace")
                setattr(target, n[2], val)


def _raise_exception(msg=""):
    raise TemplateError(str(msg))


class Prompt:
    """`Prompt` (wgml-chat/src/prompt.rs:46-108): the conversation so far."""

    def __init__(self):
        self.entries: List[Dict[str, str]] = []

    def append_user(self, text: str) -> "Prompt":
        self.entries.append({"role": "user", "content": text})
        return self

    def append_assistant(self, text: str) -> "Prompt":
        self.entries.append({"role": "assistant", "content": text})
        return self

    def append_system(self, text: str) -> "Prompt":
        self.entries.append({"role": "system", "content": text})
        return self

    def clear(self) -> None:
        self.entries.clear()

    def to_jinja_messages(self) -> List[Dict[str, str]]:
        return [dict(e) for e in self.entries]


class ChatTemplate:
    """`ChatTemplate` (wgml-chat/src/chat_template.rs:5-40)."""

    def __init__(self, template: str):
        # the reference rewrites two Python idioms its engine lacks (`.split(` -> `|split(`,
        # `[-1]` -> `|last`, chat_template.rs:11-15); both forms are understood here as they are
        self.template = template
        items = _split_source(template, trim_blocks=True)
        self._nodes, end = _parse_nodes(items, 0, ())
        if end != len(items):
            raise TemplateError("unexpected end of block")

    @classmethod
    def from_gguf(cls, gguf) -> "ChatTemplate":
        """The file's `tokenizer.chat_template`, else the Llama-2 default
        (chat_template.rs:18-25)."""
        text = gguf.metadata.get("tokenizer.chat_template") if gguf is not None else None
        return cls(text if isinstance(text, str) else LLAMA2_CHAT_TEMPLATE)

    def apply(self, prompt, bos: str, eos: str, add_generation_prompt: bool = True) -> str:
        """Renders the conversation (chat_template.rs:27-39).  `prompt`: a Prompt or a
        sequence of {"role", "content"} maps."""
        messages = prompt.to_jinja_messages() if isinstance(prompt, Prompt) else [dict(m) for m in prompt]
        env: Dict[str, Any] = {"messages": messages, "bos_token": bos, "eos_token": eos,
                               "add_generation_prompt": add_generation_prompt,
                               "raise_exception": _raise_exception,
                               "namespace": lambda **kw: _Namespace(**kw),
                               "range": lambda *a: list(range(*a))}
        out: List[str] = []
        _render(self._nodes, env, out)
        return "".join(out)
