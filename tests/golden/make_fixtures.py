#!/usr/bin/env python3
"""Transcribes golden vectors from the reference's own unit tests into JSON.

The reference's test files are read AS TEXT (nothing in them is imported or
executed): each `it(...)` spec is tokenised by the tiny expression reader below,
which understands just enough of the test idiom -- const declarations, number /
string / array / object literals, integer arithmetic, `tf.tensorNd(values,
shape)`, `tf.scalar`, the `generateCaseInputs` helper of fused_conv2d_test.ts
(restated here) and `expectArraysClose(await r.data(), [...])` -- to recover the
inputs, the op arguments and the expected outputs of a spec. Specs it cannot read
(loops, gradients, error cases) are skipped and listed.

Run in the build container, where the reference tree is mounted:
    python tests/golden/make_fixtures.py [/root/reference]
It rewrites tests/golden/*.json. The JSON files are the committed fixtures; the
tests read only those.
"""
import json
import math
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.dirname(os.path.abspath(__file__))


class Skip(Exception):
    pass


# ---------------------------------------------------------------- tokenizer
TOKEN = re.compile(r"""
    (?P<ws>\s+|//[^\n]*|/\*.*?\*/)
  | (?P<num>(?:\d+\.\d*|\.\d+|\d+)(?:[eE][-+]?\d+)?)
  | (?P<str>'[^']*'|"[^"]*"|`[^`]*`)
  | (?P<id>[A-Za-z_$][\w$]*)
  | (?P<op>=>|\.\.\.|[-+*/%(){}\[\],.:;=<>!?&|])
""", re.X | re.S)


def tokenize(src):
    pos, out = 0, []
    while pos < len(src):
        m = TOKEN.match(src, pos)
        if not m:
            raise Skip("cannot tokenize at %r" % src[pos:pos + 20])
        pos = m.end()
        kind = m.lastgroup
        if kind != "ws":
            out.append((kind, m.group()))
    return out


class Tensor:
    def __init__(self, values, shape):
        self.values = [float(v) for v in values]
        self.shape = [int(s) for s in shape]
        n = 1
        for s in self.shape:
            n *= s
        if n != len(self.values):
            raise Skip("tensor size mismatch %s vs %d" % (self.shape, len(self.values)))

    def to_json(self):
        return {"shape": self.shape, "values": self.values}


class OpCall:
    def __init__(self, op, args):
        self.op, self.args = op, args


def flatten(v):
    """Nested list -> (flat values, shape)."""
    if not isinstance(v, list):
        return [v], []
    if not v:
        return [], [0]
    flat, shape = [], None
    for e in v:
        f, s = flatten(e)
        flat += f
        shape = s
    return flat, [len(v)] + shape


GENERATOR_VARIANT = "fused"


def generate_case_inputs(total_tensor, total_filter):
    if GENERATOR_VARIANT == "conv2d":
        # conv2d_test.ts:23-35, restated: 1, 2, 3, ...
        return {"input": [i + 1 for i in range(total_tensor)],
                "filter": [i + 1 for i in range(total_filter)]}
    # fused_conv2d_test.ts:22-35, restated
    inp = [i * 0.001 - total_tensor * 0.001 / 2 for i in range(total_tensor)]
    filt = [i * 0.001 * (-1 if i % 2 == 0 else 1) for i in range(total_filter)]
    return {"input": inp, "filter": filt}


class Parser:
    def __init__(self, toks, env):
        self.t, self.i, self.env = toks, 0, env

    def peek(self, k=0):
        return self.t[self.i + k] if self.i + k < len(self.t) else ("eof", "")

    def eat(self, val=None):
        tok = self.peek()
        if val is not None and tok[1] != val:
            raise Skip("expected %r got %r" % (val, tok[1]))
        self.i += 1
        return tok

    def expr(self):
        v = self.term()
        while self.peek()[1] in ("+", "-"):
            op = self.eat()[1]
            r = self.term()
            v = v + r if op == "+" else v - r
        if self.peek() == ("id", "as"):  # TypeScript cast
            self.eat()
            self.skip_type()
        return v

    def skip_type(self):
        depth = 0
        while True:
            k, v = self.peek()
            if k == "eof":
                return
            if v in "([{<":
                depth += 1
            elif v in ")]}>":
                if depth == 0:
                    return
                depth -= 1
            elif v in (",", ";") and depth == 0:
                return
            self.eat()

    def term(self):
        v = self.unary()
        while self.peek()[1] in ("*", "/", "%"):
            op = self.eat()[1]
            r = self.unary()
            if op == "*":
                v = v * r
            elif op == "/":
                v = v / r
            else:
                v = v % r
        return v

    def unary(self):
        if self.peek()[1] == "-":
            self.eat()
            return -self.unary()
        if self.peek()[1] == "+":
            self.eat()
            return self.unary()
        return self.postfix()

    def postfix(self):
        v = self.primary()
        while True:
            nxt = self.peek()[1]
            if nxt == ".":
                self.eat()
                name = self.eat()[1]
                if isinstance(v, tuple) and name in ("data", "dataSync"):
                    self.args()
                elif isinstance(v, dict) and name in v:
                    v = v[name]
                elif isinstance(v, str) and v.startswith("@"):
                    v = v + "." + name
                else:
                    raise Skip("member %s" % name)
            elif nxt == "(" and isinstance(v, str) and v.startswith("@"):
                v = self.call(v)
            else:
                return v

    def args(self):
        self.eat("(")
        out = []
        while self.peek()[1] != ")":
            out.append(self.expr())
            if self.peek()[1] == ",":
                self.eat()
        self.eat(")")
        return out

    def call(self, fn):
        a = self.args()
        m = re.match(r"@tf\.tensor([1-6])d$", fn)
        if m or fn == "@tf.tensor":
            vals, shape = flatten(a[0])
            if len(a) > 1 and isinstance(a[1], list):
                shape = a[1]
            return Tensor(vals, shape)
        if fn == "@tf.scalar":
            return Tensor([a[0]], [])
        if fn == "@generateCaseInputs":
            return generate_case_inputs(int(a[0]), int(a[1]))
        if fn in ("@tf.fused.conv2d", "@tf.fused.matMul", "@tf.fused.depthwiseConv2d"):
            return OpCall(fn[4:], a[0])
        if fn == "@tf.conv2d":
            keys = ["x", "filter", "strides", "pad", "dataFormat", "dilations",
                    "dimRoundingMode"]
            return OpCall("conv2d", dict(zip(keys, a)))
        if fn == "@tf.depthwiseConv2d":
            keys = ["x", "filter", "strides", "pad", "dataFormat", "dilations",
                    "dimRoundingMode"]
            return OpCall("depthwiseConv2d", dict(zip(keys, a)))
        if fn == "@conv_util.computeConv2DInfo":
            keys = ["inShape", "filterShape", "strides", "dilations", "pad",
                    "roundingMode", "depthwise", "dataFormat"]
            return OpCall("computeConv2DInfo", dict(zip(keys, a)))
        if fn == "@tf.matMul":
            keys = ["a", "b", "transposeA", "transposeB"]
            return OpCall("matMul", dict(zip(keys, a)))
        raise Skip("call %s" % fn)

    def primary(self):
        k, v = self.eat()
        if k == "num":
            f = float(v)
            return int(v) if re.match(r"^\d+$", v) else f
        if k == "str":
            return v[1:-1]
        if v == "[":
            out = []
            while self.peek()[1] != "]":
                out.append(self.expr())
                if self.peek()[1] == ",":
                    self.eat()
            self.eat("]")
            return out
        if v == "{":
            out = {}
            while self.peek()[1] != "}":
                key = self.eat()[1]
                if self.peek()[1] == ":":
                    self.eat()
                    out[key] = self.expr()
                else:
                    out[key] = self.lookup(key)
                if self.peek()[1] == ",":
                    self.eat()
            self.eat("}")
            return out
        if v == "(":
            r = self.expr()
            self.eat(")")
            return r
        if k == "id":
            if v == "new":
                self.eat()  # Float32Array / Int32Array
                return self.args()[0]
            if v == "await":
                return self.unary()
            if v in ("null", "undefined"):
                return None
            if v == "true":
                return True
            if v == "false":
                return False
            if v in ("tf", "generateCaseInputs", "conv_util"):
                return "@" + v
            if v == "Math":
                raise Skip("Math")
            return self.lookup(v)
        raise Skip("unexpected token %r" % v)

    def lookup(self, name):
        if name not in self.env:
            raise Skip("unknown identifier %s" % name)
        return self.env[name]


def split_statements(body):
    """Top-level `;`-separated statements of a spec body."""
    out, depth, cur = [], 0, []
    for tok in body:
        v = tok[1]
        if v in "([{":
            depth += 1
        elif v in ")]}":
            depth -= 1
        if v == ";" and depth == 0:
            out.append(cur)
            cur = []
        else:
            cur.append(tok)
            if v == "}" and depth == 0 and cur[0][1] in ("for", "if"):
                out.append(cur)
                cur = []
    if cur:
        out.append(cur)
    return out


def strip_decl_type(toks):
    # const NAME : TYPE = ...  ->  drop TYPE (types never contain '=')
    if len(toks) > 2 and toks[2][1] == ":":
        j = 3
        while toks[j][1] != "=":
            j += 1
        return toks[:2] + toks[j:]
    return toks


def read_spec(body_src):
    toks = tokenize(body_src)
    env, cases = {}, []
    result_of = {}
    for st in split_statements(toks):
        if not st:
            continue
        head = st[0][1]
        if head in ("const", "let"):
            st = strip_decl_type(st)
            if len(st) < 4 or st[2][1] != "=":
                raise Skip("declaration form")
            name = st[1][1]
            p = Parser(st[3:], env)
            val = p.expr()
            if p.peek()[0] != "eof":
                raise Skip("trailing tokens in declaration of %s" % name)
            if isinstance(val, OpCall):
                cases.append({"call": val})
                result_of[name] = cases[-1]
                env[name] = ("@result", len(cases) - 1)
            else:
                env[name] = val
        elif head == "expect":
            # expect(x.shape).toEqual([...])
            p = Parser(st, env)
            try:
                p.eat()
                p.eat("(")
                target = p.eat()[1]
                p.eat(".")
                attr = p.eat()[1]
                while p.peek()[1] == ".":
                    p.eat()
                    attr += "." + p.eat()[1]
                p.eat(")")
                p.eat(".")
                if p.eat()[1] not in ("toEqual", "toBe"):
                    raise Skip("matcher")
                shape = p.args()[0]
                if attr == "shape" and target in result_of:
                    result_of[target]["shape"] = shape
                elif target in result_of and \
                        result_of[target]["call"].op == "computeConv2DInfo":
                    result_of[target].setdefault("fields", {})[attr] = shape
            except Skip:
                pass
        elif head == "expectArraysClose" or head == "expectArraysEqual":
            p = Parser(st[1:], env)
            a = p.args()
            got, want = a[0], a[1]
            if isinstance(got, tuple) and got[0] == "@result":
                cases[got[1]]["expected"] = want
            else:
                raise Skip("expectArraysClose on non-result")
        elif head == "for":
            run_for_loop(st, env)
        elif head == "if":
            # only `if (tf.getBackend() === ...) { return; }` guards are skipped
            if not any(t[1] == "getBackend" for t in st):
                raise Skip("control flow")
        elif head == "while":
            raise Skip("control flow")
        else:
            raise Skip("statement starts with %s" % head)
    return cases


def run_for_loop(st, env):
    """for (let i = 0; i < LIMIT; i++) { NAME.push(EXPR); ... }"""
    vals = [t[1] for t in st]
    try:
        if vals[1:6] != ["(", "let", vals[3], "=", "0"] or vals[6] != ";":
            raise Skip("for-loop header")
        var = vals[3]
        close = vals.index(")")
        header = st[7:close]
        semi = [k for k, t in enumerate(header) if t[1] == ";"][0]
        cond = header[:semi]
        if cond[0][1] != var or cond[1][1] != "<":
            raise Skip("for-loop condition")
        limit = Parser(cond[2:], env).expr()
        if vals[close + 1] != "{" or vals[-1] != "}":
            raise Skip("for-loop body")
        body = split_statements(st[close + 2:-1])
    except (IndexError, ValueError):
        raise Skip("for-loop form")
    for i in range(int(limit)):
        env[var] = i
        for b in body:
            if not b:
                continue
            if len(b) < 5 or b[1][1] != "." or b[2][1] != "push":
                raise Skip("for-loop statement")
            p = Parser(b[3:], env)
            env[b[0][1]].append(p.args()[0])
    env.pop(var, None)


def tensor_or_none(v):
    if v is None:
        return None
    if isinstance(v, Tensor):
        return v.to_json()
    raise Skip("expected a tensor")


def case_to_json(case, name, source):
    call = case["call"]
    args = call.args
    if "expected" not in case:
        raise Skip("no expected values")
    exp_vals, exp_shape = flatten(case["expected"])
    out = {"name": name, "source": source, "op": call.op}
    for k, v in args.items():
        if isinstance(v, Tensor):
            out[k] = v.to_json()
        elif isinstance(v, tuple):
            raise Skip("chained result")
        else:
            out[k] = v
    out["expected"] = {"shape": case.get("shape"),
                       "values": [float(x) for x in exp_vals]}
    for v in out["expected"]["values"]:
        if isinstance(v, float) and math.isnan(v):
            raise Skip("nan expected")
    return out


def extract_specs(path):
    """Yields (name, first_line, last_line, body_source) for each it(...)."""
    src = open(path).read()
    for m in re.finditer(r"\n\s*it\(\s*((?:'[^']*'|\s|\+)+),\s*(?:async\s*)?\(\)\s*=>\s*\{", src):
        name = "".join(re.findall(r"'([^']*)'", m.group(1)))
        start = m.end()
        depth, i = 1, start
        while depth and i < len(src):
            c = src[i]
            if c == "{":
                depth += 1
            elif c == "}":
                depth -= 1
            elif c in "'`\"":
                j = src.index(c, i + 1)
                i = j
            i += 1
        body = src[start:i - 1]
        first = src.count("\n", 0, m.start() + 1) + 1
        last = src.count("\n", 0, i) + 1
        yield name, first, last, body


def harvest_conv_info(rel_path, out_name):
    path = os.path.join(REF, rel_path)
    fixtures = []
    for name, first, last, body in extract_specs(path):
        try:
            for c in read_spec(body):
                if c["call"].op == "computeConv2DInfo" and c.get("fields"):
                    fixtures.append({"name": name,
                                     "source": "%s:%d-%d" % (rel_path, first, last),
                                     "args": c["call"].args, "expected": c["fields"]})
        except (Skip, ValueError, KeyError, IndexError, TypeError):
            pass
    with open(os.path.join(OUT, out_name), "w") as f:
        json.dump({"reference_file": rel_path, "cases": fixtures}, f, indent=0)
        f.write("\n")
    print("%-32s %3d cases" % (out_name, len(fixtures)))


def harvest(rel_path, out_name, keep_ops, exclude=()):
    global GENERATOR_VARIANT
    GENERATOR_VARIANT = "conv2d" if rel_path.endswith("/conv2d_test.ts") else "fused"
    path = os.path.join(REF, rel_path)
    fixtures, skipped = [], []
    for name, first, last, body in extract_specs(path):
        if any(e in name for e in exclude):
            continue
        try:
            cases = read_spec(body)
            got = 0
            for c in cases:
                if c["call"].op in keep_ops and "expected" in c:
                    fixtures.append(case_to_json(
                        c, name, "%s:%d-%d" % (rel_path, first, last)))
                    got += 1
            if not got:
                raise Skip("no checked op call")
        except (Skip, ValueError, KeyError, IndexError, TypeError) as e:
            skipped.append("%s:%d %s -- %s" % (os.path.basename(rel_path), first, name, e))
    with open(os.path.join(OUT, out_name), "w") as f:
        json.dump({"reference_file": rel_path, "cases": fixtures}, f, indent=0)
        f.write("\n")
    print("%-32s %3d cases, %3d specs skipped" % (out_name, len(fixtures), len(skipped)))
    return skipped


def main():
    skipped = []
    grad = ("gradient", "backProp", "throws", "grad", "upcasts", "complex")
    skipped += harvest("tfjs-core/src/ops/fused/fused_mat_mul_test.ts",
                       "fused_mat_mul.json", {"fused.matMul"}, grad)
    skipped += harvest("tfjs-core/src/ops/fused/fused_conv2d_test.ts",
                       "fused_conv2d.json", {"fused.conv2d"}, grad)
    skipped += harvest("tfjs-core/src/ops/fused/fused_depthwise_conv2d_test.ts",
                       "fused_depthwise_conv2d.json", {"fused.depthwiseConv2d"}, grad)
    skipped += harvest("tfjs-core/src/ops/mat_mul_test.ts", "mat_mul.json",
                       {"matMul"}, grad)
    skipped += harvest("tfjs-core/src/ops/conv2d_test.ts", "conv2d.json",
                       {"conv2d"}, grad)
    skipped += harvest("tfjs-core/src/ops/depthwise_conv2d_test.ts",
                       "depthwise_conv2d.json", {"depthwiseConv2d"}, grad)
    harvest_conv_info("tfjs-core/src/ops/conv_util_test.ts", "conv_util.json")
    with open(os.path.join(OUT, "SKIPPED.txt"), "w") as f:
        f.write("Specs of the reference's test files that make_fixtures.py's parser did not read, with the "
                "parser's reason (line = start of the match, which may sit a blank line above the `it(`). "
                "Where each of them is carried instead (hand_transcribed.json, tests/js/hand_specs.js, "
                "tests/js/error_specs.js) or why it is out of scope (gradient) is in spec_manifest.json.\n")
        f.write("\n".join(skipped) + "\n")

if __name__ == "__main__":
    main()
