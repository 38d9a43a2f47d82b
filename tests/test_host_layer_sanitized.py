"""The C host layer under AddressSanitizer + UndefinedBehaviorSanitizer on the CPU: `make -C skl_amd/csrc asan`
builds skl_api.c with the sanitizers, links it with the library's real objects (so the dispatch asks the real
"would this kernel take it?" predicates) and redirects everything that would reach the GPU to checking stand-ins
(tests/c/host_layer_check.c): every address range a descriptor names must lie inside the caller's buffers, every
launcher must be handed a problem it supports, and the results of random calls - every GEMM form and element kind,
fused descriptors (bias, maximum, activation, requantised copy in either orientation, q_only), the GEMM over 4-bit
weights, both pointer modes, pack / unpack, conversions, and the same calls with every scratch allocation refused -
must equal plain loops over the original arguments."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_layer_under_address_and_ub_sanitizers():
    csrc = os.path.join(ROOT, "skl_amd", "csrc")
    built = subprocess.run(["make", "-C", csrc, "../lib/host_layer_check"], capture_output=True, text=True)
    assert built.returncode == 0, built.stdout[-3000:] + built.stderr[-3000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    for args in (["900"], ["900", "0x5EED"]):   # with a seed: random cases only, without the fixed large ones
        run = subprocess.run([os.path.join(ROOT, "skl_amd", "lib", "host_layer_check")] + args, capture_output=True, text=True, env=env)
        assert run.returncode == 0, run.stdout[-3000:] + run.stderr[-6000:]
        assert "host layer ok" in run.stdout
        if len(args) == 1:   # every route of the dispatch was taken
            reached = {line.rsplit(None, 1)[0].strip(): int(line.rsplit(None, 1)[1]) for line in run.stdout.splitlines()[1:]}
            assert all(count > 0 for count in reached.values()), reached
