"""Runs TenniS operator test-case directories against device "hip": the counterpart of TenniS's own
`run_test <path> [device [id]]` (tools/run_test.cpp, tools/run_test/test_case.hpp), so that case
directories written for TenniS check this backend unchanged.

A case is a directory holding (test_case.hpp:218-246, 318-420)
    0.<op>.txt          three integers: parameter, input and output counts
    1.<param>.t         one tensor file per operator parameter
    2.input_<i>.t       the inputs
    3.output_<i>.t      the expected output (exactly one)
and passes when the operator's inferred prototype and its output's prototype equal the expected
one and max|diff| <= 1e-4, mean|diff| <= 1e-5 as fp32 (WARNING up to 10x those; test_case.hpp:468-517).
An operator the device does not register is SKIP, as in the reference.

    python -m tennis_amd.run_test <path> [device [id]]
"""
import os
import sys

import numpy as np

from . import operators, tensor_file

OK, SKIP, WARNING, FAILED = "OK", "SKIP", "WARNING", "FAILED"
MAX_MAX = 1e-4
MAX_AVG = 1e-5


class CaseError(ValueError):
    """A directory that is a test case but a broken one."""


class TestCase:
    __test__ = False   # not a pytest class

    def __init__(self):
        self.op = ""
        self.param, self.input, self.output = {}, {}, {}
        self.param_count = self.input_count = self.output_count = 0
        self.log = []

    @staticmethod
    def load(root):
        """The case in directory ``root``, or None when the directory holds no `0.<op>.txt`."""
        tc = TestCase()
        for name in sorted(os.listdir(root)):
            full = os.path.join(root, name)
            if len(name) < 5 or name[1] != "." or not os.path.isfile(full):
                continue
            if name.startswith("0.") and name.endswith(".txt"):
                with open(full) as fh:
                    words = fh.read().split()
                try:
                    tc.param_count, tc.input_count, tc.output_count = (int(w) for w in words[:3])
                except ValueError:
                    raise CaseError("format error in: " + full)
                if tc.op:
                    raise CaseError("Found two operator description in %s: %s vs. %s" % (root, name[2:-4], tc.op))
                tc.op = name[2:-4]
            elif name.startswith("1.") and name.endswith(".t"):
                tc.param[name[2:-2]] = tensor_file.read_tensor(full, with_dtype=True)
            elif name.startswith("2.input_") and name.endswith(".t"):
                tc.input[int(name[len("2.input_"):-2])] = tensor_file.read_tensor(full, with_dtype=True)
            elif name.startswith("3.output_") and name.endswith(".t"):
                tc.output[int(name[len("3.output_"):-2])] = tensor_file.read_tensor(full, with_dtype=True)
        if not tc.op:
            return None
        if len(tc.param) != tc.param_count:
            raise CaseError("Param count mismatch in %s: %d needed with %d given." % (root, tc.param_count, len(tc.param)))
        for what, have, want in (("Input", tc.input, tc.input_count), ("Output", tc.output, tc.output_count)):
            if len(have) != want:
                raise CaseError("%s count mismatch in %s: %d needed with %d given." % (what, root, want, len(have)))
            for i in range(want):
                if i not in have:
                    raise CaseError("%s missing in %s: index %d needed." % (what, root, i))
        if tc.output_count != 1:
            raise CaseError("%s: exactly one output is supported" % root)
        return tc

    def run(self, device="hip", device_id=0):
        self.log = []
        if not self.op:
            self.log.append("[ERROR]: operator is empty.")
            return FAILED
        if not operators.is_registered(device, self.op):
            self.log.append('[SKIP]: Not supported operator "%s" for %s:%d' % (self.op, device, device_id))
            return SKIP
        for v in list(self.param.values()) + list(self.input.values()) + list(self.output.values()):
            if isinstance(v, list):
                self.log.append("[SKIP]: packed tensors are not supported by this runner")
                return SKIP
        params = {k: v for k, (_, v) in self.param.items()}
        inputs = [self.input[i][1] for i in range(self.input_count)]
        want_code, want = self.output[0]
        want_proto = (want_code, tuple(np.shape(want)))
        try:
            got_proto = operators.run_op(self.op, params, inputs, device=device, device_id=device_id, infer_only=True)
        except operators.OperatorError as e:
            self.log.append("[FAILED]: %s" % e)
            return FAILED
        self.log.append("Wanted: %s" % (want_proto,))
        if tuple(got_proto) != want_proto:
            self.log.append("Infer:  %s" % (tuple(got_proto),))
            return FAILED
        try:
            got = operators.run_op(self.op, params, inputs, device=device, device_id=device_id)
        except operators.OperatorError as e:
            self.log.append("[FAILED]: %s" % e)
            return FAILED
        if got.shape != want_proto[1] or operators._NP2TS.get(got.dtype) != want_code:
            self.log.append("Run:    %s %s" % (got.dtype, got.shape))
            return FAILED
        d = np.abs(np.asarray(got, np.float32) - np.asarray(want, np.float32))
        mx = float(d.max()) if d.size else 0.0
        avg = float(d.sum(dtype=np.float32) / d.size) if d.size else 0.0
        bad = not (mx <= MAX_MAX and avg <= MAX_AVG)     # NaN differences fail
        if not bad:
            self.log.append("[OK] Diff output 0: max = %g, avg = %g" % (mx, avg))
            return OK
        if mx < MAX_MAX * 10 and avg < MAX_AVG * 10:
            self.log.append("[WARNING] Diff output 0: max = %g, avg = %g" % (mx, avg))
            return WARNING
        self.log.append("[FAILED] Diff output 0: max = %g, avg = %g" % (mx, avg))
        return FAILED


def find_cases(root):
    """Every directory below (and including) ``root``, relative to it, the reference's walk order aside."""
    out = []
    for base, dirs, _ in os.walk(root):
        dirs.sort()
        out.append(os.path.relpath(base, root))
    return out


def run_tree(root, device="hip", device_id=0, out=sys.stdout):
    """Runs every case below ``root``; returns {status: [case directories]}."""
    results = {OK: [], SKIP: [], WARNING: [], FAILED: []}
    bar = "-" * 73
    for sub in find_cases(root):
        case_root = os.path.join(root, sub)
        try:
            tc = TestCase.load(case_root)
        except (CaseError, tensor_file.TensorFileError) as e:
            print(e, file=sys.stderr)
            results[FAILED].append(sub)
            continue
        if tc is None:
            continue
        status = tc.run(device, device_id)
        results[status].append(sub)
        if status in (OK, SKIP):
            print("[%s]: %s on %s:%d" % (status, sub, device, device_id), file=out)
        else:
            print(bar, file=out)
            print("[%s]: %s on %s:%d" % (status, sub, device, device_id), file=out)
            print("\n".join(tc.log), file=out)
            print(bar, file=out)
    print("[OK]: %d, [SKIP]: %d, [WARNING]: %d, [FAILED]: %d" %
          tuple(len(results[s]) for s in (OK, SKIP, WARNING, FAILED)), file=out)
    return results


def main(argv):
    if len(argv) < 2:
        print("Usage: python -m tennis_amd.run_test path [device [id]]", file=sys.stderr)
        return 1
    device = argv[2].lower() if len(argv) > 2 else "hip"
    device_id = int(argv[3]) if len(argv) > 3 else 0
    results = run_tree(argv[1], device, device_id)
    return 1 if results[FAILED] else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
