"""Generated-C oracle for packed inference.  Test infrastructure (see oracle/__init__.py).

The reference turns a discretised net into one straight-line C function (one statement per
gate) plus a batch driver, compiles it with gcc and calls it through ctypes
(difflogic/compiled_model.py:94-239, 281-319, 342-370).  This module emits a translation
unit that computes the same function with the same exported symbols and signatures:

    void logic_gate_net(T const *inp, T *out);
    void apply_logic_gate_net(bool const *inp, int *out, size_t len);

where ``T`` is the signed C integer of ``num_bits`` bits.  The arithmetic follows the
reference step for step:

* input word for feature d of block i: sample ``b`` of the block goes to bit ``b``
  (compiled_model.py:191-198, read index ``i*F*bits + b*F + d``);
* gate statements use the 16 bitwise forms of compiled_model.py:97-128, with a cast back
  to T for 8/16-bit words (:132-135); hidden values are ``const T vN`` numbered by the
  prefix sums of the layer widths, the last layer writes ``out[j]`` (:139-164);
* per class, a ripple-carry counter over bit planes, plane 0 being the MOST significant
  (:204-219), of ``ceil(log2(out/k + 1))`` planes (:180), unpacked sample by sample into
  ``out[(i*bits + b)*k + c]`` (:222-230).

Pinned by tests/golden/compiled_*.npz: outputs of the reference's own CompiledLogicNet.
"""
import ctypes
import math
import os
import subprocess
import tempfile
import time

import numpy as np

C_TYPE = {8: "char", 16: "short", 32: "int", 64: "long long"}

_EXPR = (
    lambda a, b, z: z,
    lambda a, b, z: f"{a} & {b}",
    lambda a, b, z: f"{a} & ~{b}",
    lambda a, b, z: f"{a}",
    lambda a, b, z: f"{b} & ~{a}",
    lambda a, b, z: f"{b}",
    lambda a, b, z: f"{a} ^ {b}",
    lambda a, b, z: f"{a} | {b}",
    lambda a, b, z: f"~({a} | {b})",
    lambda a, b, z: f"~({a} ^ {b})",
    lambda a, b, z: f"~{b}",
    lambda a, b, z: f"~{b} | {a}",
    lambda a, b, z: f"~{a}",
    lambda a, b, z: f"~{a} | {b}",
    lambda a, b, z: f"~({a} & {b})",
    lambda a, b, z: f"~{z}",
)


def _zero(bits):
    return {8: "(char) 0", 16: "(short) 0", 32: "0", 64: "0LL"}[bits]


def gate_statement(bits, lhs, a, b, op):
    e = _EXPR[int(op)](a, b, _zero(bits))
    if bits in (8, 16):
        e = f"({C_TYPE[bits]}) ({e})"
    return f"\t{lhs} = {e};"


def generate_c(layers, num_inputs, num_classes, bits=64):
    """``layers``: list of (idx_a, idx_b, ops) integer sequences.  Returns C source."""
    T = C_TYPE[bits]
    widths = [len(l[0]) for l in layers]
    base = np.concatenate([[0], np.cumsum(widths[:-1])]).astype(np.int64)
    last = len(layers) - 1
    lines = ["#include <stddef.h>", "#include <stdlib.h>", "#include <stdbool.h>", "",
             f"void logic_gate_net({T} const *inp, {T} *out) {{"]
    for li, (ia, ib, ops) in enumerate(layers):
        src = (lambda j: f"inp[{j}]") if li == 0 else (lambda j, o=base[li - 1]: f"v{o + j}")
        for j, (ga, gb, op) in enumerate(zip(ia, ib, ops)):
            lhs = f"out[{j}]" if li == last else f"const {T} v{base[li] + j}"
            lines.append(gate_statement(bits, lhs, src(int(ga)), src(int(gb)), op))
    lines.append("}")

    n_last = widths[-1]
    per_class = n_last // num_classes
    planes = math.ceil(math.log2(n_last / num_classes + 1))
    one = {8: "(char) 1", 16: "(short) 1", 32: "1", 64: "1LL"}[bits]
    lines.append(f"""
void apply_logic_gate_net(bool const *inp, int *out, size_t len) {{
    enum {{ F = {num_inputs}, BITS = {bits}, NOUT = {n_last}, K = {num_classes},
           PER_CLASS = {per_class}, PLANES = {planes} }};
    {T} *words = malloc(F * sizeof({T}));
    {T} *gates = malloc(NOUT * sizeof({T}));
    {T} *count = malloc(PLANES * sizeof({T}));

    for (size_t blk = 0; blk < len; ++blk) {{
        bool const *rows = inp + blk * (size_t) F * BITS;

        /* sample s of the block -> bit s of every feature word */
        for (size_t f = 0; f < F; ++f) {{
            {T} w = {_zero(bits)};
            for (int s = BITS - 1; s >= 0; --s) {{
                w <<= 1;
                w += !!rows[(size_t) s * F + f];
            }}
            words[f] = w;
        }}

        logic_gate_net(words, gates);

        for (size_t c = 0; c < K; ++c) {{
            /* bit-sliced counter, count[0] is the most significant plane */
            for (int p = 0; p < PLANES; ++p) count[p] = {_zero(bits)};
            for (size_t n = 0; n < PER_CLASS; ++n) {{
                {T} carry = gates[c * PER_CLASS + n];
                for (int p = PLANES - 1; p >= 0; --p) {{
                    const {T} old = count[p];
                    count[p] = old ^ carry;
                    carry = old & carry;
                }}
            }}
            for (size_t s = 0; s < BITS; ++s) {{
                const {T} probe = {one} << s;
                int v = 0;
                for (int p = 0; p < PLANES; ++p) {{
                    v <<= 1;
                    v += !!(count[p] & probe);
                }}
                out[(blk * BITS + s) * K + c] = v;
            }}
        }}
    }}
    free(words);
    free(gates);
    free(count);
}}
""")
    return "\n".join(lines)


class CompiledNet:
    """gcc-compiled net, callable on a bool array [B,F] -> int32 [B,k]
    (compiled_model.py:241-319 for the build, :342-370 for the call)."""

    def __init__(self, layers, num_inputs, num_classes, bits=64, opt_level=1, compiler="gcc",
                 keep_path=None):
        self.num_inputs, self.num_classes, self.bits = num_inputs, num_classes, bits
        src = generate_c(layers, num_inputs, num_classes, bits)
        self._dir = tempfile.mkdtemp(prefix="dl_oracle_cgen_")
        c_path = os.path.join(self._dir, "net.c")
        self.lib_path = keep_path or os.path.join(self._dir, "net.so")
        with open(c_path, "w") as f:
            f.write(src)
        t0 = time.time()
        subprocess.run([compiler, "-shared", "-fPIC", f"-O{opt_level}", "-o", self.lib_path, c_path],
                       check=True)
        self.compile_seconds = time.time() - t0
        self._fn = load_apply_fn(self.lib_path)

    def __call__(self, x_bool):
        return call_apply_fn(self._fn, x_bool, self.num_classes, self.bits)


def load_apply_fn(lib_path):
    fn = ctypes.CDLL(lib_path).apply_logic_gate_net
    fn.restype = None
    fn.argtypes = [np.ctypeslib.ndpointer(ctypes.c_bool, flags="C_CONTIGUOUS"),
                   np.ctypeslib.ndpointer(ctypes.c_int32, flags="C_CONTIGUOUS"),
                   ctypes.c_size_t]
    return fn


def call_apply_fn(fn, x_bool, num_classes, bits):
    """Pads the batch with zero samples to a whole number of words, calls the library, and
    drops the pad rows (compiled_model.py:349-366)."""
    x = np.ascontiguousarray(np.asarray(x_bool, dtype=np.bool_))
    B, F = x.shape
    blocks = -(-B // bits)
    if blocks * bits != B:
        x = np.concatenate([x, np.zeros((blocks * bits - B, F), dtype=np.bool_)])
    out = np.zeros(blocks * bits * num_classes, dtype=np.int32)
    fn(x.reshape(-1), out, blocks)
    return out.reshape(blocks * bits, num_classes)[:B].copy()
