"""CompiledLogicNet: CPU inference of a trained, discretised logic-gate net through generated C
(reference: difflogic/compiled_model.py).  Same constructor, ``compile`` / ``load`` / ``forward``
API, exported symbols and numerical result as the reference; the generated C is organised
differently:

* ``mode='unrolled'`` (the reference's scheme, default below 50 000 gates): one C statement per
  gate.  gcc needs minutes for nets of several 100 000 gates (one giant function).
* ``mode='table'`` (default above): the wiring and gate ids are emitted as static tables and a
  compact interpreter loop evaluates them; compiles in well under a second at any size and runs
  at about the speed of the unrolled code built with -O0.

``num_threads`` other than 1 (0 = all cores) spreads the blocks of ``num_bits`` samples over OpenMP
threads (compiled with ``-fopenmp``); the reference's generated code is single-threaded.

Both variants export ``apply_logic_gate_net(bool const *inp, int *out, size_t len)`` with the
reference's meaning: ``inp`` holds ``len`` blocks of ``num_bits`` samples x ``num_inputs`` bools
(sample-major), ``out`` receives ``num_classes`` int32 bit counts per sample.
"""
import ctypes
import math
import os
import shutil
import subprocess
import tempfile
import time
from typing import Union

import numpy as np
import torch

from .difflogic import GroupSum, LogicLayer

_C_TYPE = {8: "signed char", 16: "short", 32: "int", 64: "long long"}
_U_TYPE = {8: "unsigned char", 16: "unsigned short", 32: "unsigned int", 64: "unsigned long long"}

# gate id -> C expression over the unsigned words a, b (truth table = binary expansion of the id)
_GATE_EXPR = ("(T) 0", "a & b", "a & ~b", "a", "b & ~a", "b", "a ^ b", "a | b", "~(a | b)", "~(a ^ b)", "~b",
              "a | ~b", "~a", "~a | b", "~(a & b)", "~(T) 0")


class CompiledLogicNet(torch.nn.Module):
    def __init__(self, model: torch.nn.Sequential, device="cpu", num_bits=64, cpu_compiler="gcc", verbose=False,
                 mode=None, num_threads=1):
        super().__init__()
        self.model = model
        self.device = device
        self.num_bits = num_bits
        self.cpu_compiler = cpu_compiler
        self.mode = mode
        self.num_threads = int(num_threads)      # 1: single-threaded like the reference; 0: all cores (OpenMP)
        assert self.num_threads >= 0, num_threads
        assert cpu_compiler in ["clang", "gcc"], cpu_compiler
        assert num_bits in [8, 16, 32, 64]
        assert mode in [None, "unrolled", "table"], mode
        self.lib_fn = None
        self._lib_dir = None
        if model is None:
            return
        assert isinstance(model[-1], GroupSum), (
            "The last layer of the model must be GroupSum, but it is {} / {} instead.".format(type(model[-1]), model[-1]))
        self.num_classes = model[-1].k
        self.num_inputs = None
        self.layers = []
        for layer in model:
            if isinstance(layer, LogicLayer):
                if self.num_inputs is None:
                    self.num_inputs = layer.in_dim
                self.num_out_per_class = layer.out_dim // self.num_classes
                self.layers.append((layer.indices[0].detach().cpu().numpy().astype(np.int64),
                                    layer.indices[1].detach().cpu().numpy().astype(np.int64),
                                    layer.weights.detach().argmax(1).cpu().numpy().astype(np.uint8)))
            elif isinstance(layer, (torch.nn.Flatten, GroupSum)):
                if verbose:
                    print("Skipping {} layer.".format(type(layer).__name__))
            else:
                assert False, "Error: layer {} / {} unknown.".format(type(layer), layer)
        assert self.layers, "the model holds no LogicLayer"
        if verbose:
            print("`layers` created and has {} layers.".format(len(self.layers)))

    # ------------------------------------------------------------------ C generation
    def _num_gates(self):
        return sum(len(l[0]) for l in self.layers)

    def _resolved_mode(self):
        if self.mode is not None:
            return self.mode
        return "unrolled" if self._num_gates() < 50_000 else "table"

    def _driver_code(self):
        T, bits = _U_TYPE[self.num_bits], self.num_bits
        n_last = len(self.layers[-1][0])
        per_class = n_last // self.num_classes
        planes = max(1, math.ceil(math.log2(n_last / self.num_classes + 1)))
        omp_region = omp_for = ""
        if self.num_threads != 1:               # every thread owns its buffers; blocks are independent
            omp_region = "#pragma omp parallel" + (f" num_threads({self.num_threads})" if self.num_threads > 1 else "")
            omp_for = "#pragma omp for schedule(static)"
        return f"""
void apply_logic_gate_net(bool const *inp, int *out, size_t len) {{
    enum {{ F = {self.num_inputs}, BITS = {bits}, NOUT = {n_last}, K = {self.num_classes},
           PER_CLASS = {per_class}, PLANES = {planes} }};
{omp_region}
    {{
    T *words = malloc(sizeof(T) * F);
    T *gates = malloc(sizeof(T) * NOUT);
{omp_for}
    for (long long blk = 0; blk < (long long) len; ++blk) {{
        bool const *rows = inp + blk * (size_t) F * BITS;
        for (size_t f = 0; f < F; ++f) {{                    /* sample s of the block -> bit s */
            T w = 0;
            for (int s = 0; s < BITS; ++s) w |= (T) (rows[(size_t) s * F + f] != 0) << s;
            words[f] = w;
        }}
        logic_gate_net(({_C_TYPE[bits]} const *) words, ({_C_TYPE[bits]} *) gates);
        for (size_t c = 0; c < K; ++c) {{                    /* bit-sliced count per class */
            T cnt[PLANES];
            for (int p = 0; p < PLANES; ++p) cnt[p] = 0;
            for (size_t n = 0; n < PER_CLASS; ++n) {{
                T carry = gates[c * PER_CLASS + n];
                for (int p = 0; p < PLANES && carry; ++p) {{
                    const T old = cnt[p];
                    cnt[p] = old ^ carry;
                    carry = old & carry;
                }}
            }}
            for (int s = 0; s < BITS; ++s) {{
                int v = 0;
                for (int p = 0; p < PLANES; ++p) v |= (int) ((cnt[p] >> s) & 1) << p;
                out[(blk * BITS + s) * K + c] = v;
            }}
        }}
    }}
    free(words);
    free(gates);
    }}
}}
"""

    def get_c_code(self):
        T = _U_TYPE[self.num_bits]
        head = ["#include <stddef.h>", "#include <stdlib.h>", "#include <stdbool.h>", "", f"typedef {T} T;", ""]
        sig = f"void logic_gate_net({_C_TYPE[self.num_bits]} const *inp_, {_C_TYPE[self.num_bits]} *out_) {{"
        body = [sig, "\tT const *inp = (T const *) inp_;", "\tT *out = (T *) out_;"]
        if self._resolved_mode() == "unrolled":
            base = 0
            for li, (ia, ib, ops) in enumerate(self.layers):
                last = li == len(self.layers) - 1
                src = (lambda j: f"inp[{j}]") if li == 0 else (lambda j, o=base - len(self.layers[li - 1][0]): f"v{o + j}")
                for j in range(len(ia)):
                    expr = _GATE_EXPR[int(ops[j])].replace("a", "@A").replace("b", "@B")
                    expr = expr.replace("@A", src(int(ia[j]))).replace("@B", src(int(ib[j])))
                    lhs = f"out[{j}]" if last else f"const T v{base + j}"
                    body.append(f"\t{lhs} = (T) ({expr});")
                base += len(ia)
            body.append("}")
            return "\n".join(head + body) + self._driver_code()
        # table mode: static wiring tables + one interpreter loop per layer
        tables, widths = [], [len(l[0]) for l in self.layers]
        for li, (ia, ib, ops) in enumerate(self.layers):
            tables.append(f"static const int A{li}[] = {{{','.join(str(int(v)) for v in ia)}}};")
            tables.append(f"static const int B{li}[] = {{{','.join(str(int(v)) for v in ib)}}};")
            tables.append(f"static const unsigned char G{li}[] = {{{','.join(str(int(v)) for v in ops)}}};")
        gate_fn = ["static inline T gate(T a, T b, unsigned op) {", "\tswitch (op) {"]
        gate_fn += [f"\tcase {i}: return (T) ({e});" for i, e in enumerate(_GATE_EXPR[:15])]
        gate_fn += ["\tdefault: return (T) ~(T) 0;", "\t}", "}", ""]
        widest = max(widths)
        # the two layer buffers are per-thread statics: no allocation per block of samples
        body += [f"\tstatic __thread T buf0[{widest}], buf1[{widest}];",
                 "\tT *cur = buf0, *nxt = buf1, *tmp;", "\tT const *src = inp;"]
        for li, w in enumerate(widths):
            dst = "out" if li == len(widths) - 1 else "nxt"
            body.append(f"\tfor (int n = 0; n < {w}; ++n) {dst}[n] = gate(src[A{li}[n]], src[B{li}[n]], G{li}[n]);")
            if li != len(widths) - 1:
                body.append("\ttmp = cur; cur = nxt; nxt = tmp; src = cur;")
        body += ["}"]
        return "\n".join(head + tables + [""] + gate_fn + body) + self._driver_code()

    # ------------------------------------------------------------------ build / load / call
    @staticmethod
    def _bind(path):
        fn = ctypes.CDLL(path).apply_logic_gate_net
        fn.restype = None
        fn.argtypes = [np.ctypeslib.ndpointer(ctypes.c_bool, flags="C_CONTIGUOUS"),
                       np.ctypeslib.ndpointer(ctypes.c_int32, flags="C_CONTIGUOUS"), ctypes.c_size_t]
        return fn

    def compile(self, opt_level=1, save_lib_path=None, verbose=False):
        """Generates the C, compiles it with ``cpu_compiler -shared -fPIC -O{opt_level}`` and binds
        ``apply_logic_gate_net``; ``save_lib_path`` keeps a copy of the shared library."""
        assert self.device == "cpu", "Device {} not supported.".format(self.device)
        code = self.get_c_code()
        # held on the object (replacing the directory of an earlier compile()) and removed with it;
        # the bound library stays usable after the file is gone
        self._lib_dir = tempfile.TemporaryDirectory(prefix="difflogic_amd_compiled_")
        c_path, so_path = os.path.join(self._lib_dir.name, "net.c"), os.path.join(self._lib_dir.name, "net.so")
        with open(c_path, "w") as f:
            f.write(code)
        if verbose:
            print("C code created ({} mode, {} lines) at {}".format(self._resolved_mode(), code.count("\n") + 1, c_path))
        t0 = time.time()
        flags = ["-shared", "-fPIC", "-O{}".format(opt_level)] + (["-fopenmp"] if self.num_threads != 1 else [])
        out = subprocess.run([self.cpu_compiler, *flags, "-o", so_path, c_path])
        if out.returncode != 0:
            raise RuntimeError(f"compilation exited with error code {out.returncode}")
        print("Compiling finished in {:.3f} seconds.".format(time.time() - t0))
        if save_lib_path is not None:
            shutil.copy(so_path, save_lib_path)
            if verbose:
                print("lib_file copied from {} to {} .".format(so_path, save_lib_path))
        self.lib_fn = self._bind(so_path)

    @staticmethod
    def load(save_lib_path, num_classes, num_bits):
        self = CompiledLogicNet(None, num_bits=num_bits)
        self.num_classes = num_classes
        self.lib_fn = CompiledLogicNet._bind(save_lib_path)
        return self

    def forward(self, x: Union[torch.BoolTensor, np.ndarray], verbose: bool = False) -> torch.IntTensor:
        """bool [B, num_inputs] -> int32 [B, num_classes]; the batch is padded with all-false
        samples to a multiple of ``num_bits`` and the pad rows are dropped again."""
        assert self.lib_fn is not None, "call compile() or load() first"
        if isinstance(x, torch.Tensor):
            x = x.cpu().numpy()
        x = np.ascontiguousarray(x, dtype=np.bool_)
        batch = x.shape[0]
        blocks = math.ceil(batch / self.num_bits)
        pad = blocks * self.num_bits - batch
        if pad:
            x = np.concatenate([x, np.zeros((pad,) + x.shape[1:], dtype=np.bool_)])
        out = np.zeros(blocks * self.num_bits * self.num_classes, dtype=np.int32)
        self.lib_fn(x.reshape(-1), out, blocks)
        out = torch.from_numpy(out).view(blocks * self.num_bits, self.num_classes)[:batch]
        if verbose:
            print("out.shape", out.shape)
        return out
