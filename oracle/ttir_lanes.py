"""TEST INFRASTRUCTURE - not part of the product.

Lane-by-lane interpreter of TTIR text in numpy: it executes a Triton program the
way the Triton language defines it - a tensor of pointers is an array of element
addresses, a mask is an array of booleans evaluated per lane, tt.load gathers and
tt.store scatters - without any notion of structured accesses.  It shares no
code with the product's planner (own reader, own evaluation), which makes it the
brute-force pin for what the reference derives symbolically:

  * addresses: lib/AnalysisStructured/PtrAnalysis.cpp (offsets, strides, sizes)
  * valid extents: lib/Analysis/MaskAnalysis.cpp:461-603 - for prefix-shaped masks
    the number of true lanes per dimension must equal dims[i], including the
    all-masked case the max() at :568-585 exists for
  * per-program results of the CPU path (serial grid, backend/driver.py:116-133).

Beyond the five hot-path kernels it also runs what the generic kernel family takes: tt.reduce / tt.scan with any
combiner region (argmin / argmax, ConversionPatterns.hpp:1443-1769), integer, bit and conversion ops, extern functions
by symbol name, tt.trans / tt.reshape / tt.cat / tt.join / tt.split, cf.cond_br trees (early return), scf.if, and block
pointers as ops (tt.make_tensor_ptr / tt.advance / boundaryCheck + padding, with the language's `0 <= index < shape` per
checked dimension; pinned by running the same kernels with the frontend's rewrite to plain pointers).  Pins, all in
tests/test_oracle_pins.py: the reference's golden tensors (python/examples/test_modulo.py, test_mask.py,
test_gather_scatter.py and the 21 cases of tests/reference_cases.py), numpy closed forms per op class
(tests/op_zoo.py, including an independent Philox for tl.rand), float64 formulas for the float kernels.

Reductions fold sequentially in index order in f32 and tt.dot sums k innermost
into a zero tile before adding the accumulator, as the reference's lowering does
(ConversionPatterns.hpp:1171-1196,1395-1407).  bf16 tensors are held as float32
arrays of exactly representable values.  Meant for small shapes: every program
is a Python-level loop over numpy calls.
"""
import re

import numpy as np

_INT_BITS = {"i1": 1, "i8": 8, "i16": 16, "i32": 32, "i64": 64, "index": 64}
_NP = {"i1": np.bool_, "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64, "index": np.int64,
       "f16": np.float16, "bf16": np.float32, "f32": np.float32, "f64": np.float64}


class Ty:
    def __init__(self, shape, elem, ptr):
        self.shape, self.elem, self.ptr = tuple(shape), elem, ptr

    @property
    def tensor(self):
        return self.shape is not None and len(self.shape) > 0 or self._is_tensor

    _is_tensor = False


def parse_type(s):
    s = s.strip()
    if s.startswith("tensor<"):
        inner = s[7:-1]
        dims = []
        while True:
            m = re.match(r"(\d+)x", inner)
            if not m:
                break
            dims.append(int(m.group(1)))
            inner = inner[m.end():]
        e = parse_type(inner)
        t = Ty(dims, e.elem, e.ptr)
        t._is_tensor = True
        return t
    if s.startswith("<tensor<"):                     # short form of a block pointer type in the custom assembly
        s = "!tt.ptr" + s
    if s.startswith("!tt.ptr<tensor<"):
        inner = parse_type(s[8:-1])
        t = Ty(inner.shape, inner.elem, True)
        t._is_tensor = True
        return t
    if s.startswith("!tt.ptr<"):
        return Ty((), s[8:-1].split(",")[0].strip(), True)
    return Ty((), s, False)


def _strip_loc(text):
    out, i, n = [], 0, len(text)
    while i < n:
        if text.startswith(" loc(", i):
            j, depth = i + 5, 1
            while depth:
                depth += {"(": 1, ")": -1}.get(text[j], 0)
                j += 1
            i = j
        else:
            out.append(text[i])
            i += 1
    return "\n".join(l for l in "".join(out).splitlines() if not l.lstrip().startswith("#loc"))


def round_bf16(x):
    """float32 array -> nearest-even bf16 value, returned as float32."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7fffffff) > 0x7f800000
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16
    r = np.where(nan, (u | 0x400000) & 0xffff0000, r).astype(np.uint32)
    return r.view(np.float32)


class BlockPtr:
    """What tt.make_tensor_ptr makes: element (i0, i1, ...) of the block is the parent's element offs[d] + i_d per dimension."""
    __slots__ = ("origin", "shape", "strides", "offs", "block")

    def __init__(self, origin, shape, strides, offs, block):
        self.origin, self.shape, self.strides, self.offs, self.block = origin, shape, strides, offs, block

    def lanes(self, checked):
        idx = np.full(self.block, self.origin, dtype=np.int64)
        mask = np.ones(self.block, dtype=bool)
        for d, (n, o, s, ext) in enumerate(zip(self.block, self.offs, self.strides, self.shape)):
            i = (o + np.arange(n, dtype=np.int64)).reshape([-1 if k == d else 1 for k in range(len(self.block))])
            idx = idx + i * s
            if d in checked:
                mask = mask & (i >= 0) & (i < ext)
        return idx, mask


class Val:
    __slots__ = ("d", "elem", "base")

    def __init__(self, d, elem, base=None):
        self.d, self.elem, self.base = d, elem, base  # base: argument index for pointers


def _wrap(v, bits):
    v &= (1 << bits) - 1
    return v - (1 << bits) if bits > 1 and v >> (bits - 1) else v


def _erf(v):
    from scipy.special import erf
    return erf(v).astype(np.asarray(v).dtype)


class Interpreter:
    def __init__(self, ttir_text):
        lines = [l.strip() for l in _strip_loc(ttir_text).splitlines() if l.strip()]
        self.lines = lines
        # every tt.func of the module: the public one is the kernel, the private ones are reached by tt.call
        self.funcs = {}
        for k, l in enumerate(lines):
            if not l.startswith("tt.func"):
                continue
            name = re.search(r"@([\w.$]+)", l).group(1)
            depth, close = 0, l.index("(")
            for close in range(l.index("("), len(l)):
                depth += {"(": 1, ")": -1}.get(l[close], 0)
                if depth == 0:
                    break
            args = []
            for a in re.split(r",\s*(?=%)", l[l.index("(") + 1:close]):
                if a.strip():
                    arg, ty = a.split(":", 1)
                    args.append((arg.strip(), parse_type(ty.split("{")[0])))
            self.funcs[name] = (args, k + 1, self._skip_block(k + 1) - 1)
            if "private" not in l[:l.index("@")]:
                self.name, self.args, self.body_start = name, args, k + 1
        self._range = self.funcs[self.name][1:]
        self._returned = []

    # ---------------------------------------------------------------- running
    def run(self, grid, arg_values, memory):
        """arg_values: per kernel argument an int/float (scalars) or None (pointers);
        memory: {arg index: flat numpy array} (uint16 storage for bf16).  Returns the
        access log: one list of (kind, arg, offsets) per program, x outermost."""
        self.mem = memory
        log = []
        gx, gy, gz = (list(grid) + [1, 1])[:3]
        for x in range(gx):
            for y in range(gy):
                for z in range(gz):
                    self.pid, self.nprog, self.acc = (x, y, z), (gx, gy, gz), []
                    env = {}
                    for i, (name, ty) in enumerate(self.args):
                        if ty.ptr:
                            env[name] = Val(0, ty.elem, base=i)
                        elif ty.elem in _INT_BITS:
                            env[name] = Val(_wrap(int(arg_values[i]), _INT_BITS[ty.elem]), ty.elem)
                        else:
                            env[name] = Val(_NP[ty.elem](arg_values[i]), ty.elem)
                    self._block(self.body_start, env)
                    log.append(self.acc)
        return log

    def _block(self, i, env):
        """Executes lines from i until the closing '}' of the block; returns (next index, yielded values)."""
        L = self.lines
        while i < len(L):
            line = L[i]
            if line == "}" or line.startswith("})"):
                return i, None
            if line.startswith("scf.yield"):
                names = re.findall(r"%[\w.#$-]+", line.split(":")[0])
                return i, [env[n] for n in names]
            if line.startswith("tt.assert"):
                i += 1
                continue
            if line.startswith("tt.return"):
                # the function ends here (an early return sits in a block of its own); a callee leaves its values behind
                self._returned = [env[n] for n in re.findall(r"%[\w.#$-]+", line.split(" : ")[0])]
                return len(L), None
            if line.startswith("^"):         # a block label reached by falling through: cannot happen in valid IR
                i += 1
                continue
            if line.startswith("cf.cond_br"):
                c, then, then_args, other, other_args = re.match(
                    r"cf\.cond_br (%[\w.#$-]+), (\^\w+)(\([^)]*\))?, (\^\w+)(\([^)]*\))?$", line).groups()
                i = self._jump(*((then, then_args) if bool(env[c].d) else (other, other_args)), env)
                continue
            if line.startswith("cf.br"):
                i = self._jump(*re.match(r"cf\.br (\^\w+)(\([^)]*\))?$", line).groups(), env)
                continue
            if line.startswith("scf.if") or re.match(r"%[\w.#$:-]+(, %[\w.#$:-]+)* = scf\.if ", line):
                i = self._if(i, env)
                continue
            i = self._op(i, env)
        return i, None

    def _jump(self, label, passed, env):
        """Branch to a block of the current function; the values in `passed` ("(%a, %b : i32, i32)") become its arguments."""
        L = self.lines
        k = next(k for k in range(*self._range) if L[k].startswith((label + ":", label + "(")))
        if passed:
            values = [env[n] for n in re.findall(r"%[\w.#$-]+", passed.split(" : ")[0])]
            for n, v in zip(re.findall(r"(%[\w.#$-]+)\s*:", L[k]), values):
                env[n] = v
        return k + 1

    def _call(self, callee, values):
        args, start, end = self.funcs[callee]
        saved, self._range, self._returned = self._range, (start, end), []
        self._block(start, {name: v for (name, _ty), v in zip(args, values)})
        self._range = saved
        return self._returned

    def _if(self, i, env):
        """scf.if without results: `scf.if %c {` ... [`} else {` ...] `}`."""
        L = self.lines
        results = []
        head = L[i]
        if head.startswith("%"):                     # %r:2 = scf.if %c -> (types) {
            lhs, head = head.split(" = ", 1)
            for r in lhs.split(","):
                r = r.strip()
                results += [f"{r.split(':')[0]}#{k}" for k in range(int(r.split(":")[1]))] if ":" in r else [r]
        m = re.match(r"scf\.if (%[\w.#$-]+)( -> .*)? \{$", head)
        take = bool(env[m.group(1)].d)
        # find the matching else / end at this nesting depth
        depth, j, els = 1, i + 1, None
        while depth:
            l = L[j]
            if l == "} else {" and depth == 1:
                els = j
            elif l.endswith("{") and not l.startswith("}"):
                depth += 1
            elif l == "}" or l.startswith("})"):
                depth -= 1
            j += 1
        end = j - 1
        if take:
            k, ys = self._block(i + 1, env) if els is None else self._run_until(i + 1, els, env)
        elif els is not None:
            k, ys = self._block(els + 1, env)
        else:
            k, ys = end, None
        if results:
            for r, y in zip(results, ys):
                env[r] = y
        return len(L) if k >= len(L) else end + 1

    def _run_until(self, i, stop, env):
        L = self.lines
        while i < stop:
            if L[i].startswith("scf.yield"):
                return i, [env[n] for n in re.findall(r"%[\w.#$-]+", L[i].split(" : ")[0])]
            if L[i].startswith("tt.return"):
                return len(L), None
            if L[i].startswith("scf.if") or re.match(r"%[\w.#$:-]+(, %[\w.#$:-]+)* = scf\.if ", L[i]):
                i = self._if(i, env)
                continue
            i = self._op(i, env)
        return i, None

    def _skip_block(self, i):
        depth = 1
        L = self.lines
        while depth:
            if L[i].endswith("{") and not L[i].startswith("}"):
                depth += 1
            if L[i] == "}" or L[i].startswith("})"):
                depth -= 1
            i += 1
        return i  # index after the closing line

    # -------------------------------------------------------------------- ops
    def _op(self, i, env):
        line = self.lines[i]
        results = []
        rest = line
        if line.startswith("%"):
            lhs, rest = line.split(" = ", 1)
            for r in lhs.split(","):
                r = r.strip()
                if ":" in r:
                    b, n = r.split(":")
                    results += [f"{b}#{k}" for k in range(int(n))]
                else:
                    results.append(r)
        m = re.match(r'"?([\w.]+)"?', rest)
        name = m.group(1)
        tail = rest[m.end():].lstrip('"').strip()

        if name == "scf.for":
            return self._for(i, results, tail, env)
        if name == "tt.reduce":
            return self._reduce(i, results, tail, env)
        if name == "tt.scan":
            return self._scan(i, results, tail, env)
        if name == "arith.constant":
            lit, ty = (tail.rsplit(" : ", 1) + ["i1"])[:2] if " : " in tail else (tail, "i1")
            env[results[0]] = self._constant(lit.strip(), parse_type(ty))
            return i + 1
        if name == "tt.call":                        # @callee(%a, %b) : (types) -> types
            callee, passed = re.match(r"@([\w.$]+)\((.*?)\)", tail).groups()
            for r, v in zip(results, self._call(callee, [env[n] for n in re.findall(r"%[\w.#$-]+", passed)])):
                env[r] = v
            return i + 1
        self._last_line = line
        head, _, types = self._split_types(tail)
        ops = [env[n] for n in re.findall(r"%[\w.#$-]+", re.sub(r"\{[^}]*\}", "", head))]
        attrs = dict(re.findall(r"(\w+) = (-?\w+)", " ".join(re.findall(r"\{([^}]*)\}", head))))
        tys = [parse_type(t) for t in re.split(r"\s*(?:->|,| to | \* )\s*", types) if t.strip()] if types else []
        words = [w for w in re.split(r"[\s,]+", re.sub(r"\{[^}]*\}", "", head)) if w and not w.startswith("%")]
        if name == "tt.split":
            env[results[0]] = Val(ops[0].d[..., 0].copy(), ops[0].elem)
            env[results[1]] = Val(ops[0].d[..., 1].copy(), ops[0].elem)
            return i + 1
        out = self._eval(name, ops, attrs, tys, words)
        if results:
            env[results[0]] = out
        return i + 1

    @staticmethod
    def _split_types(tail):
        depth = 0
        j = 0
        while j < len(tail):
            c = tail[j]
            if tail.startswith("->", j):
                j += 2
                continue
            if c in "({<[":
                depth += 1
            elif c in ")}>]":
                depth -= 1
            elif c == ":" and depth == 0:
                return tail[:j], ":", tail[j + 1:]
            j += 1
        return tail, "", ""

    def _constant(self, lit, ty):
        if lit.startswith("dense<"):
            lit = lit[6:-1]
        if ty.elem in _INT_BITS:
            v = {"true": 1, "false": 0}.get(lit)
            v = int(lit) if v is None else v
            if ty._is_tensor:
                return Val(np.full(ty.shape, v, dtype=_NP[ty.elem]), ty.elem)
            return Val(_wrap(v, _INT_BITS[ty.elem]), ty.elem)
        if lit.lower().startswith("0x"):
            bits = int(lit, 16)
            if ty.elem == "f32":
                f = np.array([bits], dtype=np.uint32).view(np.float32)[0]
            elif ty.elem == "f16":
                f = np.array([bits], dtype=np.uint16).view(np.float16)[0]
            elif ty.elem == "bf16":
                f = np.array([bits << 16], dtype=np.uint32).view(np.float32)[0]
            else:
                f = np.array([bits], dtype=np.uint64).view(np.float64)[0]
        else:
            f = float(lit)
        if ty._is_tensor:
            return Val(np.full(ty.shape, f, dtype=_NP[ty.elem]), ty.elem)
        return Val(_NP[ty.elem](f), ty.elem)

    def _eval(self, name, ops, attrs, tys, words):
        if name == "tt.get_program_id":
            return Val(self.pid["xyz".index(words[0])], "i32")
        if name == "tt.get_num_programs":
            return Val(self.nprog["xyz".index(words[0])], "i32")
        if name == "tt.make_range":
            return Val(np.arange(int(attrs["start"]), int(attrs["end"]), dtype=np.int32), "i32")
        if name == "tt.splat":
            a, shape = ops[0], tys[-1].shape
            if a.base is not None:
                return Val(np.full(shape, a.d, dtype=np.int64), a.elem, base=a.base)
            return Val(np.full(shape, a.d, dtype=_NP[a.elem]), a.elem)
        if name == "tt.trans":
            order = [int(x) for x in re.search(r"order = array<i32: ([\d, ]+)>", self._last_line).group(1).split(",")]
            a = ops[0]
            return Val(np.transpose(a.d, order).copy(), a.elem, base=a.base)
        if name == "tt.cat":
            return Val(np.concatenate([ops[0].d, ops[1].d]), ops[0].elem)
        if name == "tt.join":
            return Val(np.stack([ops[0].d, ops[1].d], axis=-1), ops[0].elem)
        if name == "tt.unsplat":
            return Val(np.asarray(ops[0].d).reshape(-1)[0], ops[0].elem)
        if name == "tt.reshape":
            a = ops[0]
            return Val(np.reshape(a.d, tys[-1].shape).copy(), a.elem, base=a.base)
        if name == "tt.expand_dims":
            return Val(np.expand_dims(ops[0].d, int(attrs["axis"])), ops[0].elem, ops[0].base)
        if name == "tt.broadcast":
            return Val(np.broadcast_to(ops[0].d, tys[-1].shape).copy(), ops[0].elem, ops[0].base)
        if name == "tt.addptr":
            p, o = ops
            if isinstance(p.d, np.ndarray):
                return Val(p.d + o.d.astype(np.int64), p.elem, p.base)
            return Val(int(p.d) + int(o.d), p.elem, p.base)
        if name == "tt.make_tensor_ptr":
            t = tys[-1]
            r = len(t.shape)
            ints = [int(o.d) for o in ops[1:]]
            return Val(BlockPtr(int(ops[0].d), ints[:r], ints[r:2 * r], ints[2 * r:], tuple(t.shape)), t.elem, ops[0].base)
        if name == "tt.advance":
            b = ops[0].d
            moved = [o + int(d.d) for o, d in zip(b.offs, ops[1:])]
            return Val(BlockPtr(b.origin, b.shape, b.strides, moved, b.block), ops[0].elem, ops[0].base)
        if name == "tt.load":
            return self._load(ops)
        if name == "tt.store":
            return self._store(ops)
        if name == "tt.dot":
            a, b, c = ops
            if a.elem in _INT_BITS:              # integer product: exact, wrapped to the accumulator's width
                wide = a.d.astype(np.int64) @ b.d.astype(np.int64) + c.d.astype(np.int64)
                return Val(wide.astype(_NP[c.elem]), c.elem)
            af, bf = a.d.astype(np.float32), b.d.astype(np.float32)
            prod = np.zeros(c.d.shape, dtype=np.float32)
            for k in range(af.shape[1]):  # k innermost per output element = this order for every (i, j)
                prod = prod + af[:, k:k + 1] * bf[k:k + 1, :]
            return Val(prod + c.d, "f32")
        return self._arith(name, ops, tys, words)

    def _storage(self, arg, elem):
        return self.mem[arg]

    def _checked_dims(self):
        m = re.search(r"boundaryCheck = array<i32(?:: ([\d, ]*))?>", self._last_line)
        return [int(x) for x in m.group(1).split(",")] if m and m.group(1) else []

    def _load(self, ops):
        p = ops[0]
        store = self._seen_as(self.mem[p.base], p.elem)
        if isinstance(p.d, BlockPtr):
            idx, mask = p.d.lanes(self._checked_dims())
            pad = re.search(r"padding = (\d)", self._last_line)
            fill = np.nan if pad and pad.group(1) == "2" else 0
            out = np.full(idx.shape, fill, dtype=_NP[p.elem])
            sel = idx[mask]
            self.acc.append(("load", p.base, np.sort(sel.ravel())))
            if sel.size:
                if sel.min() < 0 or sel.max() >= store.size:
                    raise IndexError(f"block load outside argument {p.base}: [{sel.min()}, {sel.max()}] of {store.size}")
                out[mask] = self._widen(store[sel], p.elem)
            return Val(out, p.elem)
        if not isinstance(p.d, np.ndarray):
            if len(ops) > 1 and not bool(ops[1].d):      # a scalar load under a false mask reads nothing
                return Val(ops[2].d if len(ops) > 2 else _NP[p.elem](0), p.elem)
            self.acc.append(("load", p.base, np.array([p.d], dtype=np.int64)))
            return Val(self._widen(store[p.d:p.d + 1], p.elem)[0], p.elem)
        mask = ops[1].d if len(ops) > 1 else np.ones(p.d.shape, dtype=bool)
        other = ops[2].d if len(ops) > 2 else np.zeros(p.d.shape, dtype=_NP[p.elem])
        out = np.array(np.broadcast_to(other, p.d.shape), dtype=_NP[p.elem])
        idx = p.d[mask]
        self.acc.append(("load", p.base, np.sort(idx.ravel())))
        if idx.size:
            if idx.min() < 0 or idx.max() >= store.size:
                raise IndexError(f"load outside argument {p.base}: [{idx.min()}, {idx.max()}] of {store.size}")
            out[mask] = self._widen(store[idx], p.elem)
        return Val(out, p.elem)

    def _store(self, ops):
        p, v = ops[0], ops[1]
        store = self._seen_as(self.mem[p.base], p.elem)
        if isinstance(p.d, BlockPtr):
            idx, mask = p.d.lanes(self._checked_dims())
            sel = idx[mask]
            self.acc.append(("store", p.base, np.sort(sel.ravel())))
            if sel.size:
                if sel.min() < 0 or sel.max() >= store.size:
                    raise IndexError(f"block store outside argument {p.base}")
                store[sel] = self._narrow(np.asarray(v.d)[mask], p.elem)
            return None
        if not isinstance(p.d, np.ndarray):
            if len(ops) > 2 and not bool(ops[2].d):      # a scalar store under a false mask writes nothing
                return None
            self.acc.append(("store", p.base, np.array([p.d], dtype=np.int64)))
            store[p.d] = self._narrow(np.array([v.d]), p.elem)[0]
            return None
        mask = ops[2].d if len(ops) > 2 else np.ones(p.d.shape, dtype=bool)
        idx = p.d[mask]
        self.acc.append(("store", p.base, np.sort(idx.ravel())))
        if idx.size:
            if idx.min() < 0 or idx.max() >= store.size:
                raise IndexError(f"store outside argument {p.base}")
            store[idx] = self._narrow(v.d[mask], p.elem)
        return None

    @staticmethod
    def _seen_as(store, elem):
        """An argument's memory under a pointer cast to another type of the same width: the same bytes (a numpy view)."""
        want = np.dtype(_NP[elem]) if elem != "bf16" else np.dtype(np.uint16)
        if store.dtype != want and store.dtype.itemsize == want.itemsize and elem != "i1":
            return store.view(want)
        return store

    @staticmethod
    def _widen(raw, elem):
        if elem == "bf16":
            return (raw.astype(np.uint32) << 16).view(np.float32)
        return raw

    @staticmethod
    def _narrow(vals, elem):
        if elem == "bf16":
            return (np.asarray(vals, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)
        return vals

    def _arith(self, name, ops, tys, words):
        a = ops[0]
        b = ops[1] if len(ops) > 1 else None
        scalar_int = a.elem in _INT_BITS and not isinstance(a.d, np.ndarray)
        if name in ("arith.addi", "arith.subi", "arith.muli", "arith.divsi", "arith.remsi", "arith.minsi", "arith.maxsi",
                    "arith.andi", "arith.ori", "arith.xori"):
            if scalar_int:
                x, y = int(a.d), int(b.d)
                if name == "arith.divsi":
                    r = abs(x) // abs(y) * (1 if (x < 0) == (y < 0) else -1)
                elif name == "arith.remsi":
                    r = abs(x) % abs(y) * (1 if x >= 0 else -1)
                else:
                    r = {"arith.addi": x + y, "arith.subi": x - y, "arith.muli": x * y, "arith.minsi": min(x, y),
                         "arith.maxsi": max(x, y), "arith.andi": x & y, "arith.ori": x | y, "arith.xori": x ^ y}[name]
                return Val(_wrap(r, _INT_BITS[a.elem]), a.elem)
            f = {"arith.addi": np.add, "arith.subi": np.subtract, "arith.muli": np.multiply, "arith.minsi": np.minimum,
                 "arith.maxsi": np.maximum, "arith.andi": np.bitwise_and, "arith.ori": np.bitwise_or,
                 "arith.xori": np.bitwise_xor,
                 "arith.divsi": lambda x, y: (np.trunc(x.astype(np.float64) / y)).astype(x.dtype),
                 "arith.remsi": np.fmod}[name]
            with np.errstate(over="ignore"):
                return Val(f(a.d, b.d), a.elem)
        if name in ("arith.divui", "arith.remui", "arith.shli", "arith.shrsi", "arith.shrui", "arith.minui", "arith.maxui",
                    "tt.mulhiui", "math.absi"):
            bits = _INT_BITS[a.elem]
            mask = (1 << bits) - 1
            one = lambda x, y: {  # exact integers in, the result wrapped to the type on the way out
                "arith.divui": lambda: (x & mask) // (y & mask) if (y & mask) else 0,
                "arith.remui": lambda: (x & mask) % (y & mask) if (y & mask) else 0,
                "arith.shli": lambda: x << (y & (bits - 1)),
                "arith.shrsi": lambda: x >> (y & (bits - 1)),
                "arith.shrui": lambda: (x & mask) >> (y & (bits - 1)),
                "arith.minui": lambda: min(x & mask, y & mask),
                "arith.maxui": lambda: max(x & mask, y & mask),
                "tt.mulhiui": lambda: ((x & mask) * (y & mask)) >> bits,
                "math.absi": lambda: abs(x)}[name]()
            if scalar_int:
                return Val(_wrap(one(int(a.d), int(b.d) if b is not None else 0), bits), a.elem)
            xs = np.asarray(a.d).ravel().tolist()
            ys = np.asarray(b.d).ravel().tolist() if b is not None else [0] * len(xs)
            out = np.array([_wrap(one(x, y), bits) for x, y in zip(xs, ys)], dtype=_NP[a.elem]).reshape(np.asarray(a.d).shape)
            return Val(out, a.elem)
        if name == "arith.cmpi":
            x, y = a.d, b.d
            if words[0] in ("ult", "ule", "ugt", "uge"):  # compare the unsigned readings
                u = {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}[_INT_BITS[a.elem] if a.elem != "i1" else 8]
                x, y = np.asarray(x).astype(u), np.asarray(y).astype(u)
            f = {"slt": np.less, "sle": np.less_equal, "sgt": np.greater, "sge": np.greater_equal, "eq": np.equal,
                 "ne": np.not_equal, "ult": np.less, "ule": np.less_equal, "ugt": np.greater, "uge": np.greater_equal}[words[0]]
            r = f(x, y)
            return Val(r if isinstance(a.d, np.ndarray) or isinstance(b.d, np.ndarray) else int(bool(r)), "i1")
        if name == "arith.cmpf":
            lt, gt, eq = np.less(a.d, b.d), np.greater(a.d, b.d), np.equal(a.d, b.d)
            uno = np.isnan(a.d) | np.isnan(b.d)
            r = {"oeq": eq, "one": lt | gt, "olt": lt, "ole": lt | eq, "ogt": gt, "oge": gt | eq, "ord": ~uno, "uno": uno,
                 "ueq": uno | eq, "une": ~eq, "ult": uno | lt, "ule": uno | lt | eq, "ugt": uno | gt, "uge": uno | gt | eq}[words[0]]
            return Val(r if isinstance(r, np.ndarray) else int(bool(r)), "i1")
        if name == "math.fma":
            with np.errstate(all="ignore"):
                r = (np.asarray(ops[0].d, np.float64) * np.asarray(ops[1].d, np.float64) + np.asarray(ops[2].d, np.float64))
            return self._as_float(r.astype(np.float32), a.elem, isinstance(a.d, np.ndarray), already=False)
        if name == "arith.select":
            c, x, y = ops
            if x.base is not None:               # pointers: element addresses, both sides inside one argument
                if x.base != y.base:
                    raise NotImplementedError("select between pointers into different arguments")
                return Val(np.where(c.d, x.d, y.d).astype(np.int64) if isinstance(c.d, np.ndarray) else (x.d if c.d else y.d), x.elem, x.base)
            if isinstance(c.d, np.ndarray) or isinstance(x.d, np.ndarray):
                return Val(np.where(c.d, x.d, y.d).astype(_NP[x.elem]), x.elem)
            return Val(x.d if c.d else y.d, x.elem)
        if name in ("arith.extsi", "arith.trunci", "arith.index_cast"):
            e = tys[-1].elem
            if scalar_int:
                return Val(_wrap(int(a.d), _INT_BITS[e]), e)
            return Val(a.d.astype(_NP[e]), e)
        if name == "arith.extui":
            bits = _INT_BITS[a.elem]
            e = tys[-1].elem
            if scalar_int:
                return Val(int(a.d) & ((1 << bits) - 1), e)
            return Val((a.d.astype(np.int64) & ((1 << bits) - 1)).astype(_NP[e]), e)
        e = tys[-1].elem if tys else a.elem
        if name == "tt.extern_elementwise":
            fn = re.search(r"__nv_(\w+?)f\b", " ".join(words) + " " + str(self._last_line)).group(1)
            table = {"acos": np.arccos, "acosh": np.arccosh, "asin": np.arcsin, "asinh": np.arcsinh, "atan2": np.arctan2, "atan": np.arctan,
                     "atanh": np.arctanh, "ceil": np.ceil, "cos": np.cos, "cosh": np.cosh, "erf": _erf, "exp2": np.exp2, "exp": np.exp,
                     "fabs": np.abs, "floor": np.floor, "log10": np.log10, "log1p": np.log1p, "log": np.log, "log2": np.log2, "pow": np.power,
                     "rsqrt": lambda v: 1 / np.sqrt(v), "sin": np.sin, "sinh": np.sinh, "sqrt": np.sqrt, "tan": np.tan, "tanh": np.tanh,
                     "trunc": np.trunc, "fmod": np.fmod, "expm1": np.expm1, "cbrt": np.cbrt}
            with np.errstate(all="ignore"):
                r = table[fn](*[np.asarray(o.d, dtype=np.float64) for o in ops])
            return self._as_float(np.asarray(r).astype(np.float32), a.elem, isinstance(a.d, np.ndarray), already=False)
        if name == "tt.bitcast" and ops[0].base is not None:      # a pointer cast: same addresses, another element type
            return Val(ops[0].d, tys[-1].elem, ops[0].base)
        if name in ("tt.bitcast", "arith.bitcast"):
            if (a.elem in _INT_BITS) == (e in _INT_BITS):
                return Val(a.d, e)                     # signedness only
            return Val(np.asarray(a.d).view(_NP[e]) if isinstance(a.d, np.ndarray) else np.asarray([a.d]).view(_NP[e])[0], e)
        if name == "arith.fptosi":
            with np.errstate(all="ignore"):
                return Val(np.trunc(np.asarray(a.d, dtype=np.float64)).astype(_NP[e]), e)
        if name == "arith.fptoui":
            with np.errstate(all="ignore"):
                u = {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}[_INT_BITS[e]]
                return Val(np.trunc(np.asarray(a.d, dtype=np.float64)).astype(u).astype(_NP[e]), e)
        if name == "arith.uitofp":
            u = {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}[_INT_BITS[a.elem]]
            return self._as_float(np.asarray(a.d).astype(u).astype(np.float32), e, isinstance(a.d, np.ndarray))
        if name in ("tt.clampf",):
            f_max, f_min = (np.maximum, np.minimum) if "all" in words else (np.fmax, np.fmin)
            with np.errstate(all="ignore"):
                r = f_min(f_max(a.d, ops[1].d), ops[2].d)
            return self._as_float(r, a.elem, isinstance(r, np.ndarray), already=a.elem != "bf16")
        if name == "tt.precise_sqrt":
            with np.errstate(all="ignore"):
                return self._as_float(np.sqrt(a.d), a.elem, isinstance(a.d, np.ndarray), already=a.elem != "bf16")
        if name == "tt.precise_divf":
            with np.errstate(all="ignore"):
                r = np.divide(a.d, b.d)
            return self._as_float(r, a.elem, isinstance(r, np.ndarray), already=a.elem != "bf16")
        if name == "arith.sitofp":
            v = np.asarray(a.d).astype(np.float32)
            return self._as_float(v, e, isinstance(a.d, np.ndarray))
        if name in ("arith.extf", "arith.truncf"):
            v = np.asarray(a.d, dtype=np.float32) if a.elem != "f64" else np.asarray(a.d)
            return self._as_float(v, e, isinstance(a.d, np.ndarray))
        fl = {"arith.addf": np.add, "arith.subf": np.subtract, "arith.mulf": np.multiply, "arith.divf": np.divide,
              "arith.maxnumf": np.fmax, "arith.minnumf": np.fmin, "arith.maximumf": np.maximum,
              "arith.minimumf": np.minimum}
        if name in fl:
            with np.errstate(all="ignore"):
                r = fl[name](a.d, b.d)
            return self._as_float(r, a.elem, isinstance(r, np.ndarray), already=a.elem != "bf16")
        un = {"math.exp": np.exp, "math.sqrt": np.sqrt, "math.log": np.log, "math.absf": np.abs, "arith.negf": np.negative,
              "math.exp2": np.exp2, "math.log2": np.log2, "math.rsqrt": lambda v: 1 / np.sqrt(v), "math.sin": np.sin,
              "math.cos": np.cos, "math.tanh": np.tanh, "math.floor": np.floor, "math.ceil": np.ceil, "math.erf": _erf}
        if name in un:
            with np.errstate(all="ignore"):
                r = un[name](a.d)
            return self._as_float(r, a.elem, isinstance(r, np.ndarray), already=a.elem != "bf16")
        raise NotImplementedError(f"ttir_lanes: {name}")

    @staticmethod
    def _as_float(v, elem, tensor, already=False):
        if elem == "bf16":
            v = round_bf16(np.asarray(v, dtype=np.float32))
        elif not already or np.asarray(v).dtype != _NP[elem]:
            v = np.asarray(v).astype(_NP[elem])
        return Val(v if tensor else _NP[elem if elem != "bf16" else "f32"](v), elem)

    # ------------------------------------------------------------ structured
    def _for(self, i, results, tail, env):
        m = re.match(r"(%[\w.#$-]+) = (%[\w.#$-]+) to (%[\w.#$-]+) step (%[\w.#$-]+)(.*)", tail)
        iv, lb, ub, st, rest = m.groups()
        iters = re.search(r"iter_args\((.*?)\) -> ", rest)
        names, inits = [], []
        if iters:
            for pair in re.split(r",\s*(?=%)", iters.group(1)):
                n, v = pair.split("=")
                names.append(n.strip())
                inits.append(env[v.strip()])
        cur = list(inits)
        k = int(env[lb].d)
        end = i + 1
        while k < int(env[ub].d):
            env[iv] = Val(_wrap(k, _INT_BITS[env[lb].elem]), env[lb].elem)
            for n, v in zip(names, cur):
                env[n] = v
            end, yielded = self._block(i + 1, env)
            if yielded is not None:
                cur = yielded
            k += int(env[st].d)
        close = self._skip_block(i + 1) - 1  # index of the closing '}'
        for r, v in zip(results, cur):
            env[r] = v
        return close + 1

    def _fold(self, i, results, tail, env, scan):
        """tt.reduce / tt.scan with any combiner region (argmin / argmax take two operands and a region of compares and
        selects, ConversionPatterns.hpp:1443-1769): a sequential left fold along `axis` in index order, the region
        evaluated by this interpreter on whole lines at once."""
        names = re.findall(r"%[\w.#$-]+", tail[:tail.index(")")])
        operands = [env[n] for n in names]
        axis = int(re.search(r"axis = (\d+)", tail).group(1))
        reverse = re.search(r"reverse = true", tail) is not None
        args = re.findall(r"(%[\w.#$-]+)\s*:", self.lines[i + 1])
        lo = hi = i + 2
        while not self.lines[hi].startswith(("tt.reduce.return", "tt.scan.return")):
            hi += 1
        rets = re.findall(r"%[\w.#$-]+", self.lines[hi].split(" : ")[0])
        xs = [np.moveaxis(o.d, axis, 0) for o in operands]
        order = range(xs[0].shape[0] - 1, -1, -1) if reverse else range(xs[0].shape[0])
        outs = [np.empty_like(x) for x in xs]
        acc = None
        for l in order:
            cur = [Val(x[l], o.elem) for x, o in zip(xs, operands)]
            if acc is None:
                acc = cur
            else:
                local = dict(env)
                local.update(zip(args, acc + cur))
                j = lo
                while j < hi:
                    j = self._op(j, local)
                acc = [local[r] for r in rets]
            for out, a in zip(outs, acc):
                out[l] = a.d
        for k, (r, o) in enumerate(zip(results, operands)):
            if scan:
                env[r] = Val(np.moveaxis(outs[k], 0, axis), o.elem)
            else:
                d = np.asarray(acc[k].d)
                env[r] = Val(d if d.ndim else d[()], o.elem)
        return self._skip_block(i + 1)

    def _scan(self, i, results, tail, env):
        return self._fold(i, results, tail, env, scan=True)

    def _reduce(self, i, results, tail, env):
        if tail[:tail.index(")")].count("%") > 1:
            return self._fold(i, results, tail, env, scan=False)
        operand = env[re.findall(r"%[\w.#$-]+", tail)[0]]
        axis = int(re.search(r"axis = (\d+)", tail).group(1))
        comb = re.match(r'(%[\w.#$-]+) = ([\w.]+)', self.lines[i + 2]).group(2)
        x = np.moveaxis(operand.d, axis, 0)
        if operand.elem == "f64":                # the fast paths below accumulate in f32
            return self._fold(i, results, tail, env, scan=False)
        if comb == "arith.addf" and x.ndim == 1:
            out = np.add.accumulate(x.astype(np.float32), dtype=np.float32)[-1]  # sequential fold
        elif comb == "arith.addf":
            acc = np.zeros(x.shape[1:], dtype=np.float32)
            for row in x.astype(np.float32):  # sequential, index order, f32 (f16/bf16 are promoted)
                acc = acc + row
            out = acc
        elif comb in ("arith.maxnumf", "arith.maximumf"):
            f = np.fmax if comb == "arith.maxnumf" else np.maximum
            acc = np.full(x.shape[1:], -np.inf, dtype=np.float32)
            for row in x.astype(np.float32):
                acc = f(acc, row)
            out = acc
        elif comb == "arith.addi":
            out = x.sum(axis=0, dtype=x.dtype)
        else:
            return self._fold(i, results, tail, env, scan=False)
        out = out.astype(_NP[operand.elem]) if operand.elem != "bf16" else round_bf16(out)
        env[results[0]] = Val(out if out.ndim else out[()], operand.elem)
        return self._skip_block(i + 1)
