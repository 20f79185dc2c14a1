"""Test helper: method signatures out of Rust source text (a trait, or an `impl` of it), without a Rust toolchain.

Handles what the `Backend` trait and its implementations use: plain `fn` items, and `macro_rules!` macros of one shape -- an ident,
an optional second argument, an optional `where` clause -- whose body is a `paste! { ... }` block of `fn` items named with
`[<prefix_ $name _suffix>]`.  A signature is reduced to tokens: {"name", "generics", "args": [[name, type], ...], "ret", "where",
"has_body"}; module paths are dropped (`crate::core::primitives::DeviceType` and an imported `DeviceType` are the same type)."""
import re

TOKEN = re.compile(r"[A-Za-z_][A-Za-z0-9_]*|'[a-z_]+|->|::|=>|[^\sA-Za-z0-9_]")


def strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def tokens(text):
    """Canonical token string: whitespace-free, lower-case module path prefixes removed."""
    toks = TOKEN.findall(text)
    out = []
    i = 0
    while i < len(toks):
        # drop `seg::` while seg is a lower-case module name (crate, std, core, ops, primitives ...)
        if i + 1 < len(toks) and toks[i + 1] == "::" and re.fullmatch(r"[a-z_][a-z0-9_]*", toks[i]):
            i += 2
            continue
        out.append(toks[i])
        i += 1
    return " ".join(out)


def _matching(text, start, open_ch, close_ch):
    depth = 0
    for i in range(start, len(text)):
        c = text[i]
        if c == open_ch:
            depth += 1
        elif c == close_ch:
            depth -= 1
            if depth == 0:
                return i
    raise ValueError("unbalanced " + open_ch)


def macro_bodies(text):
    """name -> text inside `paste! { ... }` of every macro_rules! in `text`."""
    out = {}
    for m in re.finditer(r"macro_rules!\s+(\w+)\s*\{", text):
        end = _matching(text, m.end() - 1, "{", "}")
        block = text[m.end():end]
        p = block.find("paste!")
        if p < 0:
            continue
        b0 = block.index("{", p)
        out[m.group(1)] = block[b0 + 1:_matching(block, b0, "{", "}")]
    return out


def expand(text):
    """`text` with every invocation `NAME!{ident [, expr] [,] [where bounds]}` of a paste-style macro defined in it replaced by the
    macro's body; the macro definitions themselves are removed."""
    bodies = macro_bodies(text)
    # remove the definitions
    for m in reversed(list(re.finditer(r"macro_rules!\s+(\w+)\s*\{", text))):
        end = _matching(text, m.end() - 1, "{", "}")
        text = text[:m.start()] + text[end + 1:]
    for name, body in bodies.items():
        pat = re.compile(re.escape(name) + r"!\s*\{([^{}]*)\}")

        def repl(m, body=body):
            arg = m.group(1).strip()
            bounds = ""
            w = re.search(r"\bwhere\b", arg)
            if w:
                bounds = arg[w.end():].strip()
                arg = arg[:w.start()].strip().rstrip(",").strip()
            parts = [a.strip() for a in arg.split(",", 1)]
            ident, code = parts[0], (parts[1] if len(parts) > 1 else "")
            b = re.sub(r"\[<([^>]*)>\]", lambda g: "".join(t.replace("$name", ident) for t in g.group(1).split()), body)
            b = re.sub(r"\$\(\s*where\s*\$\(\s*\$\w+\s*\)\+\s*\)\?", ("where " + bounds) if bounds else "", b)
            b = b.replace("$code", code).replace("$name", ident)
            return b
        text = pat.sub(repl, text)
    return text


def block_of(text, header_regex):
    """Text between the braces that follow the first match of header_regex."""
    m = re.search(header_regex, text)
    if not m:
        raise KeyError(header_regex)
    b0 = text.index("{", m.end() - 1)
    return text[b0 + 1:_matching(text, b0, "{", "}")]


def _split_top(s, sep=","):
    parts, depth, cur = [], 0, ""
    i = 0
    while i < len(s):
        c = s[i]
        if c in "([{<":
            depth += 1
        elif c in ")]}":
            depth -= 1
        elif c == ">" and not (i > 0 and s[i - 1] == "-"):
            depth -= 1
        if c == sep and depth == 0:
            parts.append(cur)
            cur = ""
        else:
            cur += c
        i += 1
    if cur.strip():
        parts.append(cur)
    return [p.strip() for p in parts if p.strip()]


def functions(block):
    """Signatures of the `fn` items at the top level of a trait / impl body (macros already expanded)."""
    out = []
    depth, i = 0, 0
    n = len(block)
    while i < n:
        c = block[i]
        if c == "{":
            depth += 1
        elif c == "}":
            depth -= 1
        elif depth == 0 and block.startswith("fn", i) and (i == 0 or not (block[i - 1].isalnum() or block[i - 1] == "_")) and i + 2 < n and block[i + 2].isspace():
            m = re.match(r"fn\s+(\w+)\s*", block[i:])
            name = m.group(1)
            j = i + m.end()
            generics = ""
            if block[j] == "<":
                # generics never contain `->`
                d, k = 0, j
                while True:
                    if block[k] == "<":
                        d += 1
                    elif block[k] == ">":
                        d -= 1
                        if d == 0:
                            break
                    k += 1
                generics = block[j + 1:k]
                j = k + 1
            j = block.index("(", j)
            pe = _matching(block, j, "(", ")")
            args_text = block[j + 1:pe]
            # the rest up to `{` or `;` outside any bracket
            k, d = pe + 1, 0
            while True:
                ch = block[k]
                if ch in "(<[":
                    d += 1
                elif ch in ")]":
                    d -= 1
                elif ch == ">" and block[k - 1] != "-":
                    d -= 1
                elif d == 0 and ch in "{;":
                    break
                k += 1
            rest = block[pe + 1:k]
            ret, where = "", ""
            w = re.search(r"\bwhere\b", rest)
            if w:
                where = rest[w.end():]
                rest = rest[:w.start()]
            r = rest.find("->")
            if r >= 0:
                ret = rest[r + 2:]
            args = []
            for a in _split_top(args_text):
                if ":" in a and not a.startswith("&self") and a != "self":
                    an, at = a.split(":", 1)
                    args.append([an.strip(), tokens(at)])
                else:
                    args.append([tokens(a), ""])
            out.append({"name": name, "generics": tokens(generics), "args": args, "ret": tokens(ret), "where": tokens(where), "has_body": block[k] == "{"})
            if block[k] == "{":
                i = _matching(block, k, "{", "}") + 1
            else:
                i = k + 1
            continue
        i += 1
    return out
