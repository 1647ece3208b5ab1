"""Seeded programs in the IR, and what they compute.

`evaluate` walks the IR text the way the reference's own walker does (sarek/sarek/Sarek_ir_interp.ml: variables by
binding id, then by name :76-91; Int32 operators :171-266 -- `shr` on non-negative operands only, where filling with
zeros and with the sign agree; statements :844-941 -- a `for` evaluates both bounds once and is inclusive :858-872),
one thread after the other; `evaluate_blocks` runs a kernel with barriers superstep by superstep.  It is a model
for tests, over the subset the generators below emit: int32 and int64 arithmetic modulo 2^32 / 2^64, floats only
where nothing is rounded, records of integers as values.

`random_program(seed)` builds a kernel over (x : int32 vector, out : int32 vector, k : int32, n : int32) in which
thread tid < n computes with int32, int64 and bool lets, mutable variables, assignments, casts between the two, `if`
statements and expressions, Stdlib.Int32's and Int64's functions (by name, and with the registry's device templates as
the front end attaches them), calls of up to two helper functions (their own lets, loops and branches, a return at
every end), `for` loops in both directions (bounds that read mutable variables the body changes among them), counted
`while` loops, blocks and arrays of the thread's own (zero to begin with), and stores into out[tid * SLOTS + j].  Names come from a small pool, parameters' names
included, so bindings hide each other all the time; every use carries the id of the binding OCaml's scoping gives
it.  Sums, products and negations overflow now and then (a linear congruential step is one of the expression forms).

`random_float_program(seed)`: float32 and float64 lets and stores whose every value both types hold exactly.
`random_block_program(seed)`: supersteps over two shared arrays.
`random_record_program(seed)`: two record types, one nested in the other, as values, in vectors and through a helper."""
import random

SLOTS = 4
INT_MIN, INT_MAX = -(1 << 31), (1 << 31) - 1


class Inexact(Exception):
    """A float program left the values float32 holds exactly."""


def _exact(v):
    import struct
    if struct.unpack("f", struct.pack("f", v))[0] != v:
        raise Inexact()
    return v


def _copy(v):
    if isinstance(v, tuple):
        return (v[0], [_copy(x) if isinstance(x, (dict, tuple)) else x for x in v[1]])
    return {k: _copy(x) if isinstance(x, (dict, tuple)) else x for k, x in v.items()}


class _Return(Exception):
    def __init__(self, value):
        self.value = value


def parse(text):
    """IR text -> nested lists of atoms."""
    import re
    tokens = re.findall(r'"[^"]*"|[()]|[^\s()"]+', text)
    pos = 0

    def node():
        nonlocal pos
        tok = tokens[pos]
        pos += 1
        if tok != "(":
            return tok
        items = []
        while tokens[pos] != ")":
            items.append(node())
        pos += 1
        return items

    tree = node()
    assert pos == len(tokens)
    return tree


def _fit(v, bits=32):
    """Int32 / Int64 arithmetic is modulo 2^32 / 2^64 (OCaml's Int32 and Int64; the device text is compiled with
    wrapping signed arithmetic)."""
    half = 1 << (bits - 1)
    return (v + half) % (1 << bits) - half


def width(e):
    """32 or 64: the integer type of an expression, from its leaves (OCaml's operators take operands of one type)."""
    head = e[0]
    if head == "i64":
        return 64
    if head == "var":
        return 64 if e[3] == "i64" else 32
    if head == "cast":
        return 64 if e[1] == "i64" else 32
    if head == "intr":
        return 64 if e[1][-1] == "Int64" else 32
    if head == "if":
        return width(e[2])
    if head in ("neg", "bitnot", "add", "sub", "mul", "div", "mod", "bitand", "bitor", "bitxor", "shl", "shr"):
        return width(e[1])
    return 32


def _trunc_div(a, b):
    q = abs(a) // abs(b)
    return q if (a < 0) == (b < 0) else -q


class Thread:
    """One thread's state: bindings by id and by name (the innermost binding of a name is the last one made), the
    vectors by name."""

    def __init__(self, arrays, index, funcs=None):
        self.by_id, self.by_name, self.arrays, self.index, self.steps = {}, {}, arrays, index, 0
        self.funcs = funcs or {}
        self.geometry = {}

    def bind(self, var, value):
        self.by_id[int(var[2])] = value
        self.by_name[var[1]] = value

    def lookup(self, var):
        vid = int(var[2])
        return self.by_id[vid] if vid in self.by_id else self.by_name[var[1]]

    def expr(self, e):
        head = e[0]
        if head in ("i32", "i64"):
            return int(e[1])
        if head in ("f32", "f64"):
            return float(e[1])
        if head == "cast":
            v = self.expr(e[2])
            if e[1] in ("f32", "f64"):                      # the float programs keep to values both float types hold
                return float(v)
            if isinstance(v, float):                        # Int32.of_float: towards zero
                v = int(v)
            return _fit(v, 64 if e[1] == "i64" else 32)     # Int64.of_int32 keeps the value, to_int32 its low 32 bits
        if head == "bool":
            return e[1] == "true"
        if head == "var":
            v = self.lookup(e)
            return _copy(v) if isinstance(v, (dict, tuple)) else v
        if head == "read":
            v = self.arrays[e[1]][self.expr(e[2])]
            if isinstance(v, dict):
                return _copy(v)
            return float(v) if isinstance(v, float) or getattr(v, "dtype", None) is not None and v.dtype.kind == "f" else int(v)
        if head == "len":
            return len(self.arrays[e[1]])
        if head == "record":                                # a value: a fresh one wherever it is bound or stored
            return {f[0]: self.expr(f[1]) for f in e[2:]}
        if head == "field":
            return self.expr(e[1])[e[2]]
        if head == "variant":                               # (constructor, payload values)
            return (e[2], [self.expr(a) for a in e[3:]])
        if head == "match":
            body = self.matching_case(self.expr(e[1]), e[2:])
            return self.expr(body)
        if head == "intr":
            name = e[2]
            if name in ("global_thread_id", "global_idx_x", "global_idx"):
                return self.index
            if name in ("thread_idx_x", "block_idx_x", "block_dim_x", "grid_dim_x"):
                return self.geometry[name]
            if e[1][-1] in ("Float32", "Float64"):          # sarek/Sarek_stdlib/Float32.ml:41-157, Sarek_float64/Float64.ml
                import math
                args = [self.expr(a) for a in e[3:] if not (isinstance(a, list) and a and a[0] == "template")]
                if name == "floor": return math.copysign(float(math.floor(args[0])), args[0]) if math.floor(args[0]) == 0 else float(math.floor(args[0]))
                if name == "ceil": return math.copysign(float(math.ceil(args[0])), args[0]) if math.ceil(args[0]) == 0 else float(math.ceil(args[0]))
                if name == "abs_float": return abs(args[0])
                if name in ("min", "max"): return min(args) if name == "min" else max(args)
                if name in ("of_int", "of_float32", "of_float64"): return float(args[0])
                if name == "to_int": return _fit(int(args[0]))
                if name in ("add", "minus", "mul"):
                    return _exact({"add": args[0] + args[1], "minus": args[0] - args[1], "mul": args[0] * args[1]}[name])
                raise KeyError(name)
            assert e[1][-1] in ("Int32", "Int64"), e        # Stdlib.Int32 / Int64 (sarek/Sarek_stdlib/Int32.ml:30-88, Int64.ml)
            bits = 64 if e[1][-1] == "Int64" else 32
            args = [self.expr(a) for a in e[3:] if not (isinstance(a, list) and a and a[0] == "template")]
            if name == "abs": return _fit(abs(args[0]), bits)
            if name == "neg": return _fit(-args[0], bits)
            if name == "lognot": return ~args[0]
            if name == "min": return min(args)
            if name == "max": return max(args)
            if name == "logxor": return args[0] ^ args[1]
            if name == "mod_int32": return args[0] - args[1] * _trunc_div(args[0], args[1])
            if name == "shift_right_logical":
                assert 0 <= args[1] < bits
                return _fit((args[0] % (1 << bits)) >> args[1], bits)
            raise KeyError(name)
        if head == "if":
            return self.expr(e[2]) if self.expr(e[1]) else self.expr(e[3])
        if head == "app":                                  # a helper: its own bindings, the value its return gives
            params, body = self.funcs[e[1][1]]
            callee = Thread(self.arrays, self.index, self.funcs)
            for p, a in zip(params, [self.expr(a) for a in e[2:]]):
                callee.bind(p, a)
            try:
                callee.stmt(body)
            except _Return as r:
                return r.value
            finally:
                self.steps += callee.steps
            raise AssertionError("a helper ended without a return")
        bits = width(e)
        if head == "neg":
            v = self.expr(e[1])
            return -v if isinstance(v, float) else _fit(-v, bits)
        if head == "bitnot":
            return ~self.expr(e[1])
        if head == "not":
            return not self.expr(e[1])
        a, b = self.expr(e[1]), self.expr(e[2])
        if isinstance(a, float) and head in ("add", "sub", "mul", "div"):
            return _exact({"add": a + b, "sub": a - b, "mul": a * b, "div": a / b if head == "div" else 0.0}[head])
        if head == "add": return _fit(a + b, bits)
        if head == "sub": return _fit(a - b, bits)
        if head == "mul": return _fit(a * b, bits)
        if head == "div": return _fit(_trunc_div(a, b), bits)
        if head == "mod": return a - b * _trunc_div(a, b)
        if head == "bitand": return a & b
        if head == "bitor": return a | b
        if head == "bitxor": return a ^ b
        if head == "shl":
            assert 0 <= b < bits
            return _fit(a << b, bits)
        if head == "shr":
            assert a >= 0 and 0 <= b < bits
            return a >> b
        if head == "lt": return a < b
        if head == "le": return a <= b
        if head == "gt": return a > b
        if head == "ge": return a >= b
        if head == "eq": return a == b
        if head == "ne": return a != b
        if head == "and": return bool(a) and bool(b)
        if head == "or": return bool(a) or bool(b)
        raise KeyError(head)

    def matching_case(self, value, cases):
        """The body of the first case that takes `value`, its pattern's variables bound by name (a pattern carries no
        ids, Sarek_ir_interp.ml:873-899)."""
        constructor, payload = value
        for case in cases:
            pattern, body = case[1], case[2]
            if pattern == "_":
                return body
            if pattern[0] == "?":
                self.by_name[pattern[1]] = value
                return body
            if pattern[0] == constructor:
                for name, v in zip(pattern[1:], payload):
                    self.by_name[name] = v
                return body
        raise AssertionError("no case matches")

    def stmt(self, s):
        head = s[0]
        self.steps += 1
        if self.steps > 2_000_000:
            raise RuntimeError("the program does not end")
        if head == "empty":
            return
        if head == "return":
            raise _Return(self.expr(s[1]))
        if head == "seq":
            for c in s[1:]:
                self.stmt(c)
        elif head == "block":
            self.stmt(s[1])
        elif head in ("let", "letmut"):
            if s[2][0] == "newarray":                       # an array of the thread's own: zeros (Sarek_ir_interp.ml:908-931)
                self.arrays = dict(self.arrays)
                self.arrays[s[1][1]] = [0] * self.expr(s[2][2])
            else:
                self.bind(s[1], self.expr(s[2]))
            self.stmt(s[3])
        elif head == "assign":
            value, target = self.expr(s[2]), s[1]
            if target[0] == "lvar":
                self.bind(target[1], value)
            elif target[0] == "lfield":                     # a field of a mutable record variable or of a vector's element
                path = []
                while target[0] == "lfield":
                    path.append(target[2])
                    target = target[1]
                holder = self.lookup(target[1]) if target[0] == "lvar" else self.arrays[target[1]][self.expr(target[2])]
                for name in reversed(path[1:]):
                    holder = holder[name]
                holder[path[0]] = value
            else:
                assert target[0] == "lelem"
                self.arrays[target[1]][self.expr(target[2])] = value
        elif head == "if":
            if self.expr(s[1]):
                self.stmt(s[2])
            elif len(s) > 3:
                self.stmt(s[3])
        elif head == "match":
            self.stmt(self.matching_case(self.expr(s[1]), s[2:]))
        elif head == "while":
            while self.expr(s[1]):
                self.stmt(s[2])
        elif head == "for":
            i, stop = self.expr(s[2]), self.expr(s[3])
            step = 1 if s[4] == "upto" else -1
            while (i <= stop) if step == 1 else (i >= stop):
                self.bind(s[1], i)
                self.stmt(s[5])
                i += step
        else:
            raise KeyError(head)


def evaluate(ir, arrays, threads):
    """Runs threads 0 .. threads-1 of the kernel's body, one after the other, on `arrays` (name -> numpy int32
    array, changed in place) and the scalar arguments given in `arrays` under their names."""
    kernel = parse(ir)
    sections = {item[0]: item for item in kernel[2:] if isinstance(item, list)}
    params = [p[1] for p in sections["params"][1:]]
    body = sections["body"][1]
    vectors = {p[1]: arrays[p[1]] for p in params if isinstance(p[3], list)}
    funcs = {f[1]: (f[2][1:], f[4]) for f in sections.get("funcs", ["funcs"])[1:]}
    for index in range(threads):
        t = Thread(vectors, index, funcs)
        for p in params:
            if not isinstance(p[3], list):
                t.bind(p, float(arrays[p[1]]) if p[3] in ("f32", "f64") else int(arrays[p[1]]))
        t.stmt(body)


class _Builder:
    POOL = ["a", "b", "c", "k", "i", "j"]          # k is a parameter's name too

    def __init__(self, rng):
        self.rng, self.next_id = rng, 10
        # name -> (id, mutable) of the binding in force; the parameters first
        self.scope = {"x": (1, False), "out": (2, False), "k": (3, False), "n": (4, False), "tid": (5, False)}
        self.vectors = {"x", "out"}
        self.counters = set()      # ids of loop counters: mutable in the IR, assigned by their loop alone
        self.wide = set()          # ids of the int64 variables
        self.local_arrays = []     # names of the thread's own arrays in scope (eight int32 each)
        self.flags = set()         # ids of the bool variables
        self.helpers = []          # (name, number of parameters) of the helper functions made so far
        self.in_helper = False     # a helper sees its parameters alone: no vector, no thread index

    def helper(self, name):
        """Text of a helper function over one or two int32 parameters whose names come from the pool: lets and
        mutable variables that hide them, loops, and a return at every end."""
        r = self.rng
        outer, self.scope, self.in_helper = self.scope, {}, True
        params = []
        for pname in r.sample(self.POOL, r.randint(1, 2)):
            self.scope[pname] = (self.next_id, False)
            params.append(self.var(pname, self.next_id, False))
            self.next_id += 1
        body = self.returning(r.randint(1, 3))
        self.scope, self.in_helper = outer, False
        self.helpers.append((name, len(params)))
        return f"(func {name} (params {' '.join(params)}) i32 {body})"

    def returning(self, depth):
        r = self.rng
        if depth == 0:
            return f"(return {self.expr(r.randint(0, 2))})"
        pick = r.randint(0, 3)
        if pick == 0:
            value = self.expr(r.randint(0, 2))
            v, body = self.bound_body(r.choice(self.POOL), False, lambda: self.returning(depth - 1))
            return f"(let {v} {value} {body})"
        if pick == 1:
            value = self.expr(r.randint(0, 2))
            v, body = self.bound_body(r.choice(self.POOL), True,
                                      lambda: f"(seq {self.stmts(min(depth, 2), r.randint(1, 2))} {self.returning(depth - 1)})")
            return f"(letmut {v} {value} {body})"
        if pick == 2:
            return f"(if {self.cond(1)} {self.returning(depth - 1)} {self.returning(depth - 1)})"
        return f"(return {self.expr(r.randint(0, 2))})"

    def var(self, name, vid, mutable):
        ty = "bool" if vid in self.flags else "i64" if vid in self.wide else "i32"
        return f"(var {name} {vid} {ty}{' mut' if mutable else ''})"

    def use(self, name):
        vid, mutable = self.scope[name]
        return self.var(name, vid, mutable)

    def ints_in_scope(self):
        return [n for n, (vid, _) in self.scope.items()
                if n not in self.vectors and vid not in self.wide and vid not in self.flags]

    def longs_in_scope(self):
        return [n for n, (vid, _) in self.scope.items() if vid in self.wide]

    def expr64(self, depth):
        """An int64 expression: Int64's operators and functions over constants of all sizes, the int64 variables in
        scope and widened int32 expressions."""
        r = self.rng
        if depth == 0:
            longs = self.longs_in_scope()
            pick = r.randint(0, 3)
            if pick == 0 or (pick == 1 and not longs):
                return f"(i64 {r.choice([0, 1, -1, 5, -7, 4294967296, -4294967297, 1 << 40, 9223372036854775807, -9223372036854775808, r.randint(-1 << 62, 1 << 62)])})"
            if pick == 1:
                return self.use(r.choice(longs))
            return f"(cast i64 {self.expr(r.randint(0, 1))})"
        a, b = self.expr64(depth - 1), self.expr64(depth - 1)
        pick = r.randint(0, 9)
        if pick == 0:
            return f"({r.choice(['add', 'sub', 'mul'])} {a} {b})"
        if pick == 1:
            return f"({r.choice(['bitand', 'bitor', 'bitxor'])} {a} {b})"
        if pick == 2:
            return f"(shl (bitand {a} (i64 1048575)) (i32 {r.randint(0, 40)}))"
        if pick == 3:
            return f"(shr (bitand {a} (i64 {(1 << 50) - 1})) (i32 {r.randint(0, 45)}))"
        if pick == 4:
            return f"({r.choice(['neg', 'bitnot'])} {a})"
        if pick == 5:
            return f"(if {self.cond(0)} {a} {b})"
        if pick == 6:
            return f"(intr (Int64) {r.choice(['min', 'max'])} {a} {b})"
        if pick == 7:
            return f"(intr (Int64) shift_right_logical {a} (i32 {r.randint(0, 63)}))"
        if pick == 8:
            return f"(add (mul {a} (i64 6364136223846793005)) (i64 1442695040888963407))"
        return f"({r.choice(['div', 'mod'])} {a} (add (bitand {b} (i64 7)) (i64 1)))"

    def small(self, e, bits=7):
        return f"(bitand {e} (i32 {(1 << bits) - 1}))"

    def expr(self, depth):
        r = self.rng
        if depth == 0:
            pick = r.randint(0, 5)
            if pick == 0:
                return f"(i32 {r.randint(-9, 12)})"
            if pick == 1 and not self.in_helper:
                return f"(read x {self.use('tid')})"
            if pick == 2 and self.local_arrays:
                return f"(read {r.choice(self.local_arrays)} {self.small(self.expr(0), 3)})"
            ints = self.ints_in_scope()                      # none when int64 lets hide a helper's every parameter
            return self.use(r.choice(ints)) if ints else f"(i32 {r.randint(-9, 12)})"
        if r.random() < 0.1:                                 # the low or the high half of an int64 value
            wide = self.expr64(depth - 1)
            return r.choice([f"(cast i32 {wide})", f"(cast i32 (intr (Int64) shift_right_logical {wide} (i32 32)))"])
        if self.helpers and r.random() < 0.15:              # (a helper calls the helpers made before it)
            name, arity = r.choice(self.helpers)
            return f"(app (var {name} 0 i32) {' '.join(self.small(self.expr(depth - 1), 6) for _ in range(arity))})"
        a, b = self.expr(depth - 1), self.expr(depth - 1)
        pick = r.randint(0, 11)
        if r.random() < 0.12:                                # Stdlib.Int32's functions, by name or with the registry's template
            pick = r.randint(0, 6)
            if pick == 0:
                return f"(intr (Int32) abs {a})"
            if pick == 1:
                return f'(intr (Int32) neg (template "(-%s)") {a})'
            if pick == 2:
                return f"(intr (Int32) {r.choice(['min', 'max'])} {a} {b})"
            if pick == 3:                                    # of a negative operand too: zeros come in from the left
                return f"(sub (intr (Int32) shift_right_logical {a} (i32 {r.randint(0, 31)})) (i32 5))"
            if pick == 4:
                return f'(intr (Sarek_stdlib Int32) mod_int32 (template "(%s %% %s)") {a} (add {self.small(b, 3)} (i32 1)))'
            if pick == 5:
                return f"(intr (Int32) lognot {a})"
            return f'(intr (Int32) shift_right_logical (template "((unsigned int)%s >> %s)") {a} (i32 {r.randint(1, 31)}))'
        if pick == 10:                                       # a linear congruential step: overflows at once
            return f"(add (mul {a} (i32 1103515245)) (i32 12345))"
        if pick == 11:
            return f"(mul {a} {b})"
        if pick == 0:
            return f"({r.choice(['add', 'sub'])} {a} {b})"
        if pick == 1:
            return f"(mul {self.small(a, 5)} {self.small(b, 5)})"
        if pick == 2:
            return f"({r.choice(['bitand', 'bitor', 'bitxor'])} {a} {b})"
        if pick == 3:
            return f"(shl {self.small(a, 10)} (i32 {r.randint(0, 5)}))"
        if pick == 4:
            return f"(shr {self.small(a, 15)} (i32 {r.randint(0, 5)}))"
        if pick == 5:
            return f"(neg {a})"
        if pick == 6:
            return f"(bitnot {a})"
        if pick == 7:
            return f"(if {self.cond(0)} {a} {b})"
        if pick == 8:
            return f"({r.choice(['div', 'mod'])} {a} (add {self.small(b, 3)} (i32 1)))"
        return f"(sub {a} {b})"

    def cond(self, depth):
        r = self.rng
        if depth > 0 and r.random() < 0.4:
            pick = r.randint(0, 2)
            if pick == 0:
                return f"(not {self.cond(depth - 1)})"
            return f"({'and' if pick == 1 else 'or'} {self.cond(depth - 1)} {self.cond(depth - 1)})"
        flags = [n for n, (vid, _) in self.scope.items() if vid in self.flags]
        if flags and r.random() < 0.3:
            return self.use(r.choice(flags))
        if r.random() < 0.15:
            return f"({r.choice(['lt', 'le', 'gt', 'ge', 'eq', 'ne'])} {self.expr64(1)} {self.expr64(1)})"
        return f"({r.choice(['lt', 'le', 'gt', 'ge', 'eq', 'ne'])} {self.expr(1)} {self.expr(1)})"

    def bound_body(self, name, mutable, make_body, counter=False, wide=False):
        """Text of a binding's declaration and the body built with the name meaning the new variable."""
        vid = self.next_id
        self.next_id += 1
        if counter:
            self.counters.add(vid)
        if wide:
            self.wide.add(vid)
        hidden = self.scope.get(name)
        self.scope[name] = (vid, mutable)
        body = make_body()
        if hidden is None:
            del self.scope[name]
        else:
            self.scope[name] = hidden
        return self.var(name, vid, mutable), body

    def assign(self, name):
        vid = self.scope[name][0]
        value = self.cond(1) if vid in self.flags else self.expr64(self.rng.randint(0, 2)) if vid in self.wide \
            else self.expr(self.rng.randint(0, 2))
        return f"(assign (lvar {self.use(name)}) {value})"

    def store(self):
        if self.local_arrays and self.rng.random() < 0.4:
            return (f"(assign (lelem {self.rng.choice(self.local_arrays)} {self.small(self.expr(1), 3)}) "
                    f"{self.expr(self.rng.randint(0, 2))})")
        if self.in_helper:                                  # no memory there: an assignment, or nothing
            mutables = [n for n, (vid, m) in self.scope.items() if m and vid not in self.counters]
            if not mutables:
                return "(empty)"
            return self.assign(self.rng.choice(mutables))
        slot = self.rng.randrange(SLOTS)
        return f"(assign (lelem out (add (mul {self.use('tid')} (i32 {SLOTS})) (i32 {slot}))) {self.expr(self.rng.randint(0, 2))})"

    def stmts(self, depth, count):
        return "(seq " + " ".join(self.stmt(depth) for _ in range(count)) + ")" if count != 1 else self.stmt(depth)

    def stmt(self, depth):
        r = self.rng
        mutables = [n for n, (vid, m) in self.scope.items() if m and vid not in self.counters]
        if depth == 0:
            if mutables and r.random() < 0.5:
                return self.assign(r.choice(mutables))
            return self.store()
        pick = r.randint(0, 9)
        if pick in (0, 1, 2, 3):                             # let [mutable] NAME = e in S (the value reads the outer NAME)
            if r.random() < 0.12:                            # a bool: the name stands for a condition from here on
                value = self.cond(1)
                vid = self.next_id
                self.flags.add(vid)
                v, body = self.bound_body(r.choice(self.POOL), pick >= 2, lambda: self.stmts(depth - 1, r.randint(1, 3)))
                assert f" {vid} bool" in v
                return f"({'letmut' if pick >= 2 else 'let'} {v} {value} {body})"
            wide = r.random() < 0.25
            value = self.expr64(r.randint(0, 2)) if wide else self.expr(r.randint(0, 2))
            v, body = self.bound_body(r.choice(self.POOL), pick >= 2, lambda: self.stmts(depth - 1, r.randint(1, 3)), wide=wide)
            return f"({'letmut' if pick >= 2 else 'let'} {v} {value} {body})"
        if pick == 4:
            other = f" {self.stmts(depth - 1, r.randint(1, 2))}" if r.random() < 0.6 else ""
            return f"(if {self.cond(1)} {self.stmts(depth - 1, r.randint(1, 2))}{other})"
        if pick in (5, 6):                                   # for NAME = lo to / downto hi
            lo, hi = self.small(self.expr(1), 2), self.small(self.expr(1), 3)
            down = r.random() < 0.4
            narrow = [n for n in mutables if self.scope[n][0] not in self.wide and self.scope[n][0] not in self.flags]
            moving = r.choice(narrow) if narrow and r.random() < 0.5 else None
            if moving:                                       # the far bound reads what the body goes on to change
                bound = self.small(self.use(moving), 3)
                lo, hi = (bound, hi) if down else (lo, bound)
            first, last = (hi, lo) if down else (lo, hi)
            counter = r.choice(self.POOL)

            def turns():
                body = self.stmts(depth - 1, r.randint(1, 2))
                if moving and self.scope.get(moving, (None, False))[1] and counter != moving:
                    shown = ""
                    if not self.in_helper:
                        slot = f"(add (mul {self.use('tid')} (i32 {SLOTS})) (i32 {r.randrange(SLOTS)}))"
                        shown = f"(assign (lelem out {slot}) (add {self.use(counter)} {self.use(moving)})) "
                    body = f"(seq {body} {shown}(assign (lvar {self.use(moving)}) {self.expr(1)}))"
                return body
            # the counter is declared mutable in the IR (Sarek_lower_ir.ml:476-484) though no kernel assigns it
            v, body = self.bound_body(counter, True, turns, counter=True)
            return f"(for {v} {first} {last} {'downto' if down else 'upto'} {body})"
        if pick == 7:                                        # let lim = e in letmut turn = 0 in while turn < lim do S; turn++
            limit = self.small(self.expr(1), 3)

            def counter():
                def loop():
                    turn = self.use("turn")
                    inner = self.stmts(depth - 1, r.randint(1, 2))
                    return (f"(while (lt {turn} {self.use('lim')}) (seq {inner} "
                            f"(assign (lvar {turn}) (add {turn} (i32 1)))))")
                v, body = self.bound_body("turn", True, loop, counter=True)
                return f"(letmut {v} (i32 0) {body})"
            lim, body = self.bound_body("lim", False, counter)
            return f"(let {lim} {limit} {body})"
        if pick == 8:
            return f"(block {self.stmts(depth - 1, r.randint(1, 3))})"
        if pick == 9 and r.random() < 0.6:                   # an array of the thread's own: eight zeros to begin with
            vid = self.next_id
            self.next_id += 1
            name = f"arr{vid}"
            self.local_arrays.append(name)
            body = self.stmts(depth - 1, r.randint(2, 4))
            self.local_arrays.remove(name)
            return f"(let (var {name} {vid} (array i32 local)) (newarray i32 (i32 8) local) {body})"
        return self.store()


def random_program(seed, threads=24):
    """(ir, x, k) of the seed; out is to be SLOTS * threads elements."""
    import numpy as np
    rng = random.Random(seed * 1000)
    b = _Builder(rng)
    funcs = " ".join(b.helper(f"helper{h}") for h in range(rng.randint(0, 2)))
    body = b.stmts(rng.randint(2, 4), rng.randint(2, 4))
    ir = ("(kernel sarek_kern (params (param (var x 1 (vec i32))) (param (var out 2 (vec i32))) "
          "(param (var k 3 i32)) (param (var n 4 i32))) (locals) (body (let (var tid 5 i32) "
          f"(intr (Std) global_thread_id) (if (lt (var tid 5 i32) (var n 4 i32)) {body}))) "
          f"(funcs {funcs}) (native_fn true))")
    x = np.array([rng.randint(-100, 100) for _ in range(threads)], np.int32)
    return ir, x, rng.randint(-5, 9)


def expected(ir, x, k, threads):
    import numpy as np
    out = np.full(SLOTS * threads, -1, np.int32)
    evaluate(ir, {"x": x.copy(), "out": out, "k": k, "n": threads}, threads)
    return out


class _Floats:
    """Float programs whose every value is a multiple of 1/8 below 2^15 in size, so that float32 and float64 hold it
    exactly and a fused multiply-add gives what a multiplication and an addition give: sums and differences of
    leaves, products with powers of two, negations, conditionals, floor / ceil / abs, conversions
    between int32, float32 and float64.  Lets of both float types hide each other as in the integer programs."""
    POOL = ["a", "b", "c", "s"]            # s is a parameter's name too

    def __init__(self, rng):
        self.rng, self.next_id = rng, 10
        self.scope = {"s": (3, "f32")}     # name -> (id, type); the vectors and n are used by name below

    def use(self, name):
        vid, ty = self.scope[name]
        return f"(var {name} {vid} {ty})", ty

    def leaf(self, ty):
        r = self.rng
        names = [n for n, (_, t) in self.scope.items() if t == ty]
        pick = r.randint(0, 4)
        if pick == 0 and names:
            return self.use(r.choice(names))[0]
        if pick == 1:
            read = "(read x (var tid 5 i32))"
            return read if ty == "f32" else f"(intr (Float64) of_float32 {read})"
        if pick == 2:
            return f"(cast {ty} (bitand (var tid 5 i32) (i32 31)))"
        if pick == 3:
            other = "f64" if ty == "f32" else "f32"
            names = [n for n, (_, t) in self.scope.items() if t == other]
            if names:
                return f"(cast {ty} {self.use(r.choice(names))[0]})"
        return f"({ty} {r.randint(-64, 64) / 8})"

    def expr(self, ty, depth):
        r = self.rng
        if depth == 0:
            return self.leaf(ty)
        a, b = self.expr(ty, depth - 1), self.expr(ty, depth - 1)
        module = "Float32" if ty == "f32" else "Float64"
        pick = r.randint(0, 9)
        if pick <= 1:
            return f"({r.choice(['add', 'sub'])} {a} {b})"
        if pick == 2:
            return f"(mul {a} ({ty} {r.choice([0.5, 2.0, -1.0, 0.25, 4.0, 1.0, -2.0])}))"
        if pick == 3:
            return f"(neg {a})"
        if pick == 4:
            return f"(if ({r.choice(['lt', 'le', 'gt', 'ge', 'eq', 'ne'])} {a} {b}) {a} {b})"
        if pick == 5:
            return f"(intr ({module}) {r.choice(['floor', 'ceil', 'abs_float'])} {a})"
        if pick == 6:                                        # (no min / max: which of -0 and +0 is the smaller is nobody's law)
            return f"(if (lt {a} {b}) {b} {a})"
        if pick == 7:                                        # through int32 and back: towards zero
            return f"(intr ({module}) of_int (cast i32 {a}))"
        if pick == 8:
            return f"(div {a} ({ty} {r.choice([2.0, 4.0, -2.0, 0.5])}))"
        return f'(intr ({module}) add (template "(%s + %s)") {a} {b})'

    def body(self, lets):
        r = self.rng
        if lets == 0:
            stores = []
            for slot in range(SLOTS):
                ty = r.choice(["f32", "f64"])
                value = self.expr(ty, r.randint(0, 2))
                target = "out" if ty == "f32" else "wide"
                stores.append(f"(assign (lelem {target} (add (mul (var tid 5 i32) (i32 {SLOTS})) (i32 {slot}))) {value})")
            return "(seq " + " ".join(stores) + ")"
        ty = r.choice(["f32", "f64"])
        value = self.expr(ty, r.randint(0, 2))
        name, vid = r.choice(self.POOL), self.next_id
        self.next_id += 1
        hidden = self.scope.get(name)
        self.scope[name] = (vid, ty)
        inner = self.body(lets - 1)
        if hidden is None:
            del self.scope[name]
        else:
            self.scope[name] = hidden
        return f"(let (var {name} {vid} {ty}) {value} {inner})"


def random_float_program(seed, threads=24):
    """(ir, x, s) over (x : float32 vector, out : float32 vector, s : float32, wide : float64 vector, n : int32):
    thread tid < n stores SLOTS values into out or wide (a slot left alone keeps what the vector held)."""
    import numpy as np
    for attempt in range(100):                              # the first candidate whose every value float32 holds exactly
        rng = random.Random(500000 + seed * 100 + attempt)
        b = _Floats(rng)
        body = b.body(rng.randint(2, 6))
        ir = ("(kernel sarek_kern (params (param (var x 1 (vec f32))) (param (var out 2 (vec f32))) (param (var s 3 f32)) "
              "(param (var wide 6 (vec f64))) (param (var n 4 i32))) (locals) (body (let (var tid 5 i32) "
              f"(intr (Std) global_thread_id) (if (lt (var tid 5 i32) (var n 4 i32)) {body}))) (native_fn true))")
        x = np.array([rng.randint(-64, 64) / 8 for _ in range(threads)], np.float32)
        s = rng.randint(-32, 32) / 8
        try:
            expected_floats(ir, x, s, threads)
        except Inexact:
            continue
        return ir, x, s
    raise RuntimeError(f"seed {seed}: no exact candidate")


def expected_floats(ir, x, s, threads):
    import numpy as np
    out, wide = np.full(SLOTS * threads, -1, np.float32), np.full(SLOTS * threads, -1, np.float64)
    evaluate(ir, {"x": x.copy(), "out": out, "wide": wide, "s": s, "n": threads}, threads)
    return out, wide


def evaluate_blocks(ir, arrays, block, grid):
    """Runs a kernel of the shape `let <shared arrays and thread-private bindings> in (seq S1 (barrier) S2 ...)` block
    by block: the bindings in front of the sequence per thread, then the statements between two barriers for every
    thread of the block in turn (a superstep: the programs below read only what an earlier superstep wrote and
    write only their own slots, so the order of the threads inside one does not matter -- Sarek_cpu_runtime.ml:686-782
    runs them in that order too)."""
    kernel = parse(ir)
    sections = {item[0]: item for item in kernel[2:] if isinstance(item, list)}
    params = [p[1] for p in sections["params"][1:]]
    vectors = {p[1]: arrays[p[1]] for p in params if isinstance(p[3], list)}
    for b in range(grid):
        shared = dict(vectors)
        threads = []
        for t in range(block):
            th = Thread(shared, b * block + t)
            th.geometry = {"thread_idx_x": t, "block_idx_x": b, "block_dim_x": block, "grid_dim_x": grid}
            for p in params:
                if not isinstance(p[3], list):
                    th.bind(p, int(arrays[p[1]]))
            threads.append(th)
        # the bindings in front of the sequence: shared arrays once per block, the rest per thread
        node = sections["body"][1]
        while node[0] in ("let", "letmut"):
            if node[2][0] == "newarray":
                assert node[2][3] == "shared"
                shared[node[1][1]] = [0] * threads[0].expr(node[2][2])
            else:
                for th in threads:
                    th.bind(node[1], th.expr(node[2]))
            node = node[3]
        assert node[0] == "seq"
        for statement in node[1:]:
            if statement[0] == "barrier":
                continue
            for th in threads:
                th.stmt(statement)


def random_block_program(seed, block=64, grid=3):
    """(ir, x, k): supersteps over two shared int32 arrays of one element per thread.  A superstep writes the
    thread's own slot of one array (and, now and then, its running value) from its running value, its indices and
    slots of the arrays written in earlier supersteps, at seeded offsets and strides round the block; the last one
    stores the running value to out[global id]."""
    import numpy as np
    rng = random.Random(900000 + seed)
    tid, gid = "(var tid 10 i32)", "(var gid 11 i32)"
    acc = "(var acc 12 i32 mut)"
    arrays = ["tile", "other"]
    written = set()

    def slot_of(other_thread):
        return f"(mod (add (mul {tid} (i32 {rng.choice([1, 1, 3, 5, 7])})) (i32 {other_thread})) (intr (Gpu) block_dim_x))"

    def value(depth):
        if depth == 0:
            pick = rng.randint(0, 5)
            if pick == 0 and written:
                return f"(read {rng.choice(sorted(written))} {slot_of(rng.randint(0, 63))})"
            return [acc, tid, gid, f"(i32 {rng.randint(-9, 9)})", "(var k 3 i32)", "(intr (Gpu) block_idx_x)"][pick]
        a, b = value(depth - 1), value(depth - 1)
        op = rng.choice(["add", "sub", "mul", "bitxor", "bitand", "bitor"])
        return f"({op} {a} {b})" if op != "mul" else f"(mul (bitand {a} (i32 255)) (bitand {b} (i32 255)))"

    steps = []
    for _ in range(rng.randint(2, 6)):
        target = rng.choice(arrays)
        # a superstep may read the array it is about to overwrite only through the running value it took before
        readable = written - {target}
        saved, written_now = written, readable
        written = readable
        body = [f"(assign (lelem {target} {tid}) {value(rng.randint(1, 2))})"]
        if rng.random() < 0.6:
            body.append(f"(assign (lvar {acc}) {value(rng.randint(1, 2))})")
        written = saved | {target}
        rng.shuffle(body)
        steps.append(f"(block (seq {' '.join(body)}))" if rng.random() < 0.5 else " ".join(body))
        steps.append("(barrier)")
    final = value(2)
    steps.append(f"(assign (lelem out {gid}) {final})")
    body = (f"(let (var tile 20 (array i32 shared)) (newarray i32 (intr (Gpu) block_dim_x) shared) "
            f"(let (var other 21 (array i32 shared)) (newarray i32 (i32 {block}) shared) "
            f"(let {tid} (intr (Gpu) thread_idx_x) (let {gid} (intr (Std) global_thread_id) "
            f"(letmut {acc} (read x {gid}) (seq {' '.join(steps)}))))))")
    ir = ("(kernel sarek_kern (params (param (var x 1 (vec i32))) (param (var out 2 (vec i32))) (param (var k 3 i32))) "
          f"(locals) (body {body}) (native_fn true))")
    x = np.array([rng.randint(-100, 100) for _ in range(block * grid)], np.int32)
    return ir, x, rng.randint(-5, 9)


POINT = "(record point (x i32) (y i32))"
SEG = f"(record seg (a {POINT}) (b {POINT}) (w i32))"
SHAPE = f"(variant shape (Dot {POINT}) (Line {SEG}) (Scaled i32 i32) (Nothing))"


class _Records:
    """Programs over two record types, point {x; y} and seg {a : point; b : point; w}: record literals, elements of
    record vectors, fields and fields of fields, conditionals between records, a helper that takes a seg and returns a
    point, mutable record variables whose fields are assigned, stores of whole records and of single fields into the
    vectors; and a variant over them (Dot of point | Line of seg | Scaled of int32 * int32 | Nothing) built by
    constructors and conditionals and taken apart by matches, as statements and as values, with wildcard and variable
    patterns.  Records are values here as in the device text; no variable is bound to another mutable record (an
    alias in OCaml, a copy in C)."""

    def __init__(self, rng):
        self.rng, self.next_id = rng, 40
        self.points, self.segs, self.mutable = [], [], set()      # variables in scope, as IR text
        self.shapes, self.ints = [], []

    def shape(self, depth):
        """A value of shape = Dot of point | Line of seg | Scaled of int32 * int32 | Nothing."""
        r = self.rng
        pick = r.randint(0, 5)
        if pick == 0 and self.shapes:
            return r.choice(self.shapes)
        if pick == 1:
            return f"(variant shape Dot {self.point(depth)})"
        if pick == 2:
            return f"(variant shape Line {self.seg(max(depth - 1, 0))})"
        if pick == 3:
            return f"(variant shape Scaled {self.integer(1)} {self.integer(1)})"
        if pick == 4 and depth > 0:
            return f"(if (ne {self.integer(1)} {self.integer(1)}) {self.shape(depth - 1)} {self.shape(depth - 1)})"
        return "(variant shape Nothing)"

    def cases(self, make_body):
        """Cases over shape in a seeded order, the last one a wildcard, a variable pattern or the constructor left;
        `make_body` builds a case's body with the pattern's variables in scope."""
        r = self.rng
        constructors = ["Dot", "Line", "Scaled", "Nothing"]
        r.shuffle(constructors)
        texts = []
        for c in constructors[:r.randint(2, 4)]:
            n = self.next_id
            self.next_id += 4
            if c == "Dot":
                v = f"(var pat{n} {n} {POINT})"
                self.points.append(v)
                texts.append(f"(case (Dot pat{n}) {make_body()})")
                self.points.remove(v)
            elif c == "Line":
                v = f"(var pat{n} {n} {SEG})"
                self.segs.append(v)
                texts.append(f"(case (Line pat{n}) {make_body()})")
                self.segs.remove(v)
            elif c == "Scaled":
                a, b = f"(var pat{n} {n} i32)", f"(var pat{n + 1} {n + 1} i32)"
                self.ints += [a, b]
                texts.append(f"(case (Scaled pat{n} pat{n + 1}) {make_body()})")
                self.ints.remove(a)
                self.ints.remove(b)
            else:
                texts.append(f"(case (Nothing) {make_body()})")
        if len(texts) < 4:
            if r.random() < 0.5:
                texts.append(f"(case _ {make_body()})")
            else:
                n = self.next_id
                self.next_id += 1
                v = f"(var rest{n} {n} {SHAPE})"
                self.shapes.append(v)
                texts.append(f"(case (? rest{n}) {make_body()})")
                self.shapes.remove(v)
        return " ".join(texts)

    def fresh(self, name, ty, mutable=False):
        vid = self.next_id
        self.next_id += 1
        text = f"(var {name}{vid} {vid} {ty}{' mut' if mutable else ''})"
        if mutable:
            self.mutable.add(text)
        return text

    def integer(self, depth):
        r = self.rng
        if depth > 0 and r.random() < 0.2:                   # a match used as a value
            scrutinee = self.shape(1)
            return f"(match {scrutinee} {self.cases(lambda: self.integer(depth - 1))})"
        if depth == 0:
            pick = r.randint(0, 5)
            if self.ints and r.random() < 0.3:
                return r.choice(self.ints)
            if pick == 0:
                return f"(i32 {r.randint(-20, 20)})"
            if pick == 1:
                return "(var tid 5 i32)"
            if pick == 2 and self.segs:
                return f"(field {r.choice(self.segs)} w)"
            if pick == 3 and self.segs:
                return f"(field (field {r.choice(self.segs)} {r.choice('ab')}) {r.choice('xy')})"
            if pick == 4:
                return f"(field (read ps (var tid 5 i32)) {r.choice('xy')})"
            return f"(field {self.point(0)} {r.choice('xy')})"
        a, b = self.integer(depth - 1), self.integer(depth - 1)
        return f"({r.choice(['add', 'sub', 'bitxor', 'bitand'])} {a} {b})"

    def point(self, depth):
        r = self.rng
        pick = r.randint(0, 6)
        if pick == 0 and self.points:
            return r.choice(self.points)
        if pick == 1:
            return "(read ps (var tid 5 i32))"
        if pick == 2 and self.segs:
            return f"(field {r.choice(self.segs)} {r.choice('ab')})"
        if pick == 3:
            return f"(field (read ss (var tid 5 i32)) {r.choice('ab')})"
        if pick == 4 and depth > 0:
            return f"(if (lt {self.integer(1)} {self.integer(1)}) {self.point(depth - 1)} {self.point(depth - 1)})"
        if pick == 5 and depth > 0:
            return f"(app (var mid 0 {POINT}) {self.seg(depth - 1)})"
        return f"(record point (x {self.integer(min(depth, 1))}) (y {self.integer(min(depth, 1))}))"

    def seg(self, depth):
        r = self.rng
        pick = r.randint(0, 3)
        if pick == 0 and self.segs:
            return r.choice(self.segs)
        if pick == 1:
            return "(read ss (var tid 5 i32))"
        if pick == 2 and depth > 0:
            return f"(if (ge {self.integer(1)} {self.integer(1)}) {self.seg(depth - 1)} {self.seg(depth - 1)})"
        return f"(record seg (a {self.point(depth)}) (b {self.point(depth)}) (w {self.integer(1)}))"

    def body(self, steps):
        r = self.rng
        if steps == 0:
            stores = [f"(assign (lelem out (add (mul (var tid 5 i32) (i32 {SLOTS})) (i32 {slot}))) {self.integer(2)})" for slot in range(SLOTS)]
            stores.append(f"(assign (lelem ps (var tid 5 i32)) {self.point(2)})")
            stores.append(r.choice([f"(assign (lelem ss (var tid 5 i32)) {self.seg(1)})",
                                    f"(assign (lfield (lelem ss (var tid 5 i32)) w) {self.integer(2)})",
                                    f"(assign (lfield (lfield (lelem ss (var tid 5 i32)) {r.choice('ab')}) {r.choice('xy')}) {self.integer(2)})"]))
            r.shuffle(stores)
            return "(seq " + " ".join(stores) + ")"
        pick = r.randint(0, 6)
        if pick == 5:                                        # let v = <shape> in ...
            value, v = self.shape(2), self.fresh("v", SHAPE)
            self.shapes.append(v)
            inner = self.body(steps - 1)
            self.shapes.remove(v)
            return f"(let {v} {value} {inner})"
        if pick == 6:                                        # match <shape> with cases that store, then the rest
            slot = r.randrange(SLOTS)
            store = lambda: f"(assign (lelem out (add (mul (var tid 5 i32) (i32 {SLOTS})) (i32 {slot}))) {self.integer(1)})"
            scrutinee = self.shape(1)
            return f"(seq (match {scrutinee} {self.cases(store)}) {self.body(steps - 1)})"
        if pick <= 1:                                        # let p = <point> in ...
            value, v = self.point(2), self.fresh("p", POINT)
            self.points.append(v)
            inner = self.body(steps - 1)
            self.points.remove(v)
            return f"(let {v} {value} {inner})"
        if pick == 2:
            value, v = self.seg(1), self.fresh("s", SEG)
            self.segs.append(v)
            inner = self.body(steps - 1)
            self.segs.remove(v)
            return f"(let {v} {value} {inner})"
        # let mutable q = <literal or element> in q.f <- e; ...   (never another variable: no aliases)
        wide = pick == 4
        saved_points, saved_segs = self.points, self.segs
        self.points, self.segs = [], []                       # the initial value names no variable
        value = (self.seg(0) if wide else self.point(0))
        self.points, self.segs = saved_points, saved_segs
        v = self.fresh("q", SEG if wide else POINT, mutable=True)
        target = f"(lvar {v})"
        if wide:
            assign = r.choice([f"(assign (lfield {target} w) {self.integer(1)})",
                               f"(assign (lfield (lfield {target} {r.choice('ab')}) {r.choice('xy')}) {self.integer(1)})",
                               f"(assign (lfield {target} {r.choice('ab')}) {self.point(1)})"])
            self.segs.append(v)
        else:
            assign = f"(assign (lfield {target} {r.choice('xy')}) {self.integer(1)})"
            self.points.append(v)
        inner = self.body(steps - 1)
        (self.segs if wide else self.points).remove(v)
        return f"(letmut {v} {value} (seq {assign} {inner}))"


def random_record_program(seed, threads=24):
    """(ir, ps, ss): ps an int32 array [threads, 2], ss one [threads, 5] (a.x a.y b.x b.y w)."""
    import numpy as np
    rng = random.Random(700000 + seed)
    b = _Records(rng)
    body = b.body(rng.randint(2, 5))
    s = f"(var s 30 {SEG})"
    mid = (f"(func mid (params {s}) {POINT} (return (record point (x (add (field (field {s} a) x) (field (field {s} b) x))) "
           f"(y (sub (field (field {s} a) y) (field {s} w))))))")
    ir = (f"(kernel sarek_kern (params (param (var ps 1 (vec {POINT}))) (param (var ss 2 (vec {SEG}))) "
          "(param (var out 3 (vec i32))) (param (var n 4 i32))) (locals) (body (let (var tid 5 i32) "
          f"(intr (Std) global_thread_id) (if (lt (var tid 5 i32) (var n 4 i32)) {body}))) "
          f"(types (point (x i32) (y i32)) (seg (a {POINT}) (b {POINT}) (w i32))) "
          f"(variants (shape (Dot {POINT}) (Line {SEG}) (Scaled i32 i32) (Nothing))) (funcs {mid}) (native_fn true))")
    ps = np.array([[rng.randint(-50, 50) for _ in range(2)] for _ in range(threads)], np.int32)
    ss = np.array([[rng.randint(-50, 50) for _ in range(5)] for _ in range(threads)], np.int32)
    return ir, ps, ss


def expected_records(ir, ps, ss, threads):
    import numpy as np
    points = [{"x": int(p[0]), "y": int(p[1])} for p in ps]
    segs = [{"a": {"x": int(q[0]), "y": int(q[1])}, "b": {"x": int(q[2]), "y": int(q[3])}, "w": int(q[4])} for q in ss]
    out = np.full(SLOTS * threads, -1, np.int32)
    evaluate(ir, {"ps": points, "ss": segs, "out": out, "n": threads}, threads)
    return (np.array([[p["x"], p["y"]] for p in points], np.int32),
            np.array([[q["a"]["x"], q["a"]["y"], q["b"]["x"], q["b"]["y"], q["w"]] for q in segs], np.int32), out)
