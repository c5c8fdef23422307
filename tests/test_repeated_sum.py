"""csrc/repeated_sum.h on the host: the value of `n` in-place additions of one weight, as the
reference's homogeneous scatter loops leave it (event_csr_matvec.py:313-331,
lib/cpu_event_sum.cc:5-24), computed in closed form, against the loop itself: every bit, for
weights of any magnitude and sign, exact ties, subnormals, overflow and sums long enough to
stop moving."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_closed_form_equals_the_loop_bit_for_bit(tmp_path):
  exe = str(tmp_path / "repeated_sum_check")
  subprocess.run(["g++", "-O2", "-std=c++17", os.path.join(HERE, "repeated_sum_check.cc"), "-o", exe], check=True)
  r = subprocess.run([exe], stdout=subprocess.PIPE, text=True)
  assert r.returncode == 0, r.stdout
  assert "float: 300 cases, 0 differ" in r.stdout and "double: 200 cases, 0 differ" in r.stdout
