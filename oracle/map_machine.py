"""TEST INFRASTRUCTURE ONLY -- numpy execution of a ``NineToothedMapProgram``.

Nothing in the product imports this module.  It runs the two stack programs
that :mod:`ninetoothed_amd.mapping` produces (same opcodes and semantics as
the interpreter kernel in ``ninetoothed_amd/csrc/map.hip``) on host arrays, all
output elements at once, so that the lowering of index maps and expressions
can be checked without a GPU against :func:`oracle.programs.tile_map`, which
restates the reference's semantics independently (offset tables, not index
arithmetic).
"""

import numpy as np

from ninetoothed_amd import mapping, runtime

_NUMPY = {
    "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64, "u8": np.uint8, "u16": np.uint16,
    "u32": np.uint32, "u64": np.uint64, "fp16": np.float16, "fp32": np.float32, "fp64": np.float64,
}


def _round_bf16(values):
    as_f32 = np.asarray(values, dtype=np.float32)
    bits = as_f32.view(np.uint32)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    return np.where(np.isnan(as_f32), as_f32, rounded.view(np.float32)).astype(np.float64)


def round_to(values, dtype_index):
    tag = runtime.DATA_TYPES[dtype_index]
    if tag == "bf16":
        return _round_bf16(values)
    if tag == "fp64":
        return values
    if tag.startswith("fp"):
        with np.errstate(over="ignore"):
            return values.astype(_NUMPY[tag]).astype(np.float64)
    return np.trunc(values).astype(np.int64).astype(_NUMPY[tag]).astype(np.float64)


def philox_uniform(seed, offset):
    """Philox-4x32-10 as Triton's ``tl.rand(seed, offset)`` applies it."""
    seed = np.asarray(seed, dtype=np.int64).astype(np.uint64)
    offset = np.asarray(offset, dtype=np.int64).astype(np.uint64)
    c0 = (offset & 0xFFFFFFFF).astype(np.uint64)
    c1 = (offset >> np.uint64(32)).astype(np.uint64)
    c2 = np.zeros_like(c0)
    c3 = np.zeros_like(c0)
    k0 = np.broadcast_to(seed & np.uint64(0xFFFFFFFF), c0.shape).astype(np.uint64)
    k1 = np.broadcast_to(seed >> np.uint64(32), c0.shape).astype(np.uint64)
    a, b, mask = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57), np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0, p2 = c0, c2
        c0 = ((b * p2) >> np.uint64(32)) ^ c1 ^ k0
        c2 = ((a * p0) >> np.uint64(32)) ^ c3 ^ k1
        c1 = (b * p2) & mask
        c3 = (a * p0) & mask
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    x = c0.astype(np.uint32).view(np.int32).astype(np.int64)
    x = np.where(x < 0, -x - 1, x)
    return (x.astype(np.float32) * np.float32(4.6566127342e-10)).astype(np.float64)


def _floor_div(a, c):
    return np.floor_divide(a, c)


class Machine:
    def __init__(self, program, arrays):
        """``arrays[slot]``: flat numpy array (or a bf16 array held as float32 with
        ``bf16_slots`` naming it) of operand ``slot``."""
        self.p = program
        self.arrays = arrays

    def run_index(self, segment, variables):
        p = self.p
        stack = []
        valid = np.ones(variables[0].shape if variables else (), dtype=bool)
        pc = p.segment_begin[segment]
        while True:
            word = p.index_code[pc]
            op, arg = word & 0xFF, word >> 8
            pc += 1
            if op == mapping.I_END:
                return (stack[-1] if stack else np.zeros(valid.shape, dtype=np.int64)), valid
            if op == mapping.I_CONST:
                stack.append(np.full(valid.shape, p.index_constants[arg], dtype=np.int64))
            elif op == mapping.I_VAR:
                stack.append(variables[arg].astype(np.int64))
            elif op == mapping.I_MULC:
                stack[-1] = stack[-1] * p.index_constants[arg]
            elif op == mapping.I_ADD:
                b = stack.pop()
                stack[-1] = stack[-1] + b
            elif op == mapping.I_DIVC:
                stack[-1] = _floor_div(stack[-1], p.index_constants[arg])
            elif op == mapping.I_MODC:
                c = p.index_constants[arg]
                stack[-1] = stack[-1] - _floor_div(stack[-1], c) * c
            elif op == mapping.I_CHECK:
                v = stack.pop()
                valid &= (v >= 0) & (v < p.index_constants[arg])
            else:
                raise ValueError(f"unknown index opcode {op}")

    def run_value(self, begin, end, variables, initial=None, reduced=()):
        p = self.p
        V = mapping.V
        names = {index: name for name, index in V.items()}
        stack = [] if initial is None else [initial]
        shape = variables[0].shape if variables else ()
        with np.errstate(all="ignore"):
            for pc in range(begin, end):
                word = p.value_code[pc]
                op, arg = names[word & 0xFF], word >> 8
                if op == "LOAD":
                    operand = p.operands[arg]
                    offset, valid = self.run_index(operand.segment, variables)
                    data = self.arrays[arg]
                    safe = np.where(valid, offset, 0)
                    stack.append(np.where(valid, data[safe].astype(np.float64), operand.other))
                elif op == "CONST":
                    stack.append(np.full(shape, p.value_constants[arg], dtype=np.float64))
                elif op == "OFFSET":
                    offset, _ = self.run_index(arg, variables)
                    stack.append(offset.astype(np.float64))
                elif op in ("ADD", "SUB", "MUL", "DIV", "FLOORDIV", "MOD", "POW", "MAX", "MIN", "LT", "LE", "GT", "GE", "EQ", "NE", "AND", "OR"):
                    b = stack.pop()
                    a = stack.pop()
                    stack.append({
                        "ADD": lambda: a + b, "SUB": lambda: a - b, "MUL": lambda: a * b, "DIV": lambda: a / b,
                        "FLOORDIV": lambda: np.floor(a / b), "MOD": lambda: a - np.floor(a / b) * b,
                        "POW": lambda: np.power(a.astype(np.float32), b.astype(np.float32)).astype(np.float64),
                        "MAX": lambda: np.maximum(a, b), "MIN": lambda: np.minimum(a, b),
                        "LT": lambda: (a < b) * 1.0, "LE": lambda: (a <= b) * 1.0, "GT": lambda: (a > b) * 1.0,
                        "GE": lambda: (a >= b) * 1.0, "EQ": lambda: (a == b) * 1.0, "NE": lambda: (a != b) * 1.0,
                        "AND": lambda: ((a != 0) & (b != 0)) * 1.0, "OR": lambda: ((a != 0) | (b != 0)) * 1.0,
                    }[op]())
                elif op == "WHERE":
                    b = stack.pop()
                    a = stack.pop()
                    c = stack.pop()
                    stack.append(np.where(c != 0, a, b))
                elif op == "ROUND":
                    stack[-1] = round_to(stack[-1], arg)
                elif op == "RAND":
                    offset = stack.pop()
                    seed = stack.pop()
                    stack.append(philox_uniform(seed.astype(np.int64), offset.astype(np.int64)))
                elif op == "SETVAR":
                    variables[arg] = np.broadcast_to(np.trunc(stack.pop()).astype(np.int64), shape)
                elif op == "REDUCED":
                    stack.append(reduced[arg])
                else:
                    a = stack.pop()
                    f32 = a.astype(np.float32)
                    stack.append({
                        "NEG": lambda: -a, "NOT": lambda: (a == 0) * 1.0, "ABS": lambda: np.abs(a),
                        "EXP": lambda: np.exp(f32).astype(np.float64), "EXP2": lambda: np.exp2(f32).astype(np.float64),
                        "LOG": lambda: np.log(f32).astype(np.float64), "LOG2": lambda: np.log2(f32).astype(np.float64),
                        "SQRT": lambda: np.sqrt(a), "RSQRT": lambda: (1 / np.sqrt(f32)).astype(np.float64),
                        "SIGMOID": lambda: (1 / (1 + np.exp(-f32))).astype(np.float64), "TANH": lambda: np.tanh(f32).astype(np.float64),
                        "SIN": lambda: np.sin(f32).astype(np.float64), "COS": lambda: np.cos(f32).astype(np.float64),
                        "FLOOR": lambda: np.floor(a), "CEIL": lambda: np.ceil(a),
                    }[op]())
        return stack[-1]

    def run_tiles(self):
        """Tile mode: whole-tile reductions as phases, then the stored expression on every element."""
        p = self.p
        grid_extents = [p.extents[v] for v in range(p.num_grid)]
        tile_extents = [p.extents[v] for v in range(p.num_grid, p.num_vars)]
        tiles = int(np.prod(grid_extents)) if grid_extents else 1
        elements = int(np.prod(tile_extents)) if tile_extents else 1
        if tiles == 0 or elements == 0:
            return
        tile_number, element_number = np.divmod(np.arange(tiles * elements), elements)
        variables = [np.asarray(g) for g in (np.unravel_index(tile_number, grid_extents) if grid_extents else ())]
        variables += [np.asarray(g) for g in (np.unravel_index(element_number, tile_extents) if tile_extents else ())]
        reduced = []
        begin = 0
        for k in range(p.num_phases):
            term = np.broadcast_to(self.run_value(begin, p.phase_end[k], variables, reduced=reduced), (tiles * elements,)).reshape(tiles, elements)
            if p.phase_op[k] == 3:
                result = round_to(term.sum(axis=1), p.phase_dtype[k])  # any summation order is as good as the kernel's tree
            elif p.phase_op[k] == 1:
                result = term.max(axis=1)
            else:
                result = term.min(axis=1)
            reduced.append(np.repeat(result, elements))
            begin = p.phase_end[k]
        value = self.run_value(begin, p.value_code_length, variables, reduced=reduced)
        self._store(value, variables)

    def run(self):
        p = self.p
        if p.num_phases:
            return self.run_tiles()
        num_out = p.num_vars - p.num_reduced
        out_extents = [p.extents[v] for v in range(num_out)]
        total = int(np.prod(out_extents)) if out_extents else 1
        if total == 0:
            return
        grids = np.unravel_index(np.arange(total), out_extents) if out_extents else ()
        variables = [np.asarray(g) for g in grids] + [None] * p.num_reduced + [np.zeros(total, dtype=np.int64)] * p.num_dynamic
        if p.reduce_op == 0:
            value = self.run_value(0, p.value_code_length, variables)
        else:
            reduced_extents = [p.extents[v] for v in range(num_out, p.num_vars)]
            acc = np.full(total, 0.0 if p.reduce_op == 3 else (-np.inf if p.reduce_op == 1 else np.inf))
            for position in np.ndindex(*reduced_extents):
                for v, index in enumerate(position):
                    variables[num_out + v] = np.full(total, index)
                term = self.run_value(0, p.reduce_split, variables)
                if p.reduce_op == 3:
                    acc = round_to(acc + term, p.reduce_dtype)
                elif p.reduce_op == 1:
                    acc = np.maximum(acc, term)
                else:
                    acc = np.minimum(acc, term)
            value = self.run_value(p.reduce_split, p.value_code_length, variables, initial=acc)
        self._store(value, variables)

    def _store(self, value, variables):
        p = self.p
        out = p.operands[p.output]
        offset, valid = self.run_index(out.segment, variables)
        target = self.arrays[p.output]
        value = np.broadcast_to(value, valid.shape)
        tag = runtime.DATA_TYPES[out.dtype]
        if tag.startswith("fp") or tag == "bf16":
            stored = value[valid].astype(target.dtype)
        else:
            stored = np.trunc(value[valid]).astype(np.int64).astype(target.dtype)
        if p.store_op == 1:  # atomic add: every output element adds its value
            np.add.at(target, offset[valid], stored)
        else:
            target[offset[valid]] = stored
