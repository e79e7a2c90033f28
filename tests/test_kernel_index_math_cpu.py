"""Runs the exact kernel bodies and launch planning on the CPU (tests/emul), every
(workgroup, lane) pair in sequence under AddressSanitizer, against the C oracle."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_kernel_bodies_match_oracle_on_cpu():
    emul = os.path.join(HERE, "emul")
    subprocess.check_call(["make", "-s", "-B", "-C", emul, "emul_check"])
    proc = subprocess.run([os.path.join(emul, "emul_check")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert " 0 failures" in proc.stdout, proc.stdout[-2000:]
