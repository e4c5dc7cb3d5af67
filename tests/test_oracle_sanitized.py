"""The CPU oracle under AddressSanitizer + UndefinedBehaviorSanitizer (`make -C oracle asan`, CPU only).

The oracle restates Rust whose integer widths decide results (a u16 shifted before it is widened, `as i8`, usize
arithmetic on short inputs).  oracle/sanitize_driver.c runs every oracle function over heap buffers of exactly the stated
size -- whole, ragged and empty inputs, all 65 536 f16 patterns, all 256 exponents and codes -- and stops on a read or
write past an end, a shift beyond a type's width or a signed overflow.  The same driver built without the sanitizers
must print the same checksum over all results."""
import os
import subprocess

ORACLE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")


def test_oracle_is_clean_under_asan_and_ubsan():
    subprocess.run(["make", "-C", ORACLE, "asan"], check=True, stdout=subprocess.DEVNULL)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0",
               UBSAN_OPTIONS="print_stacktrace=1", OMP_NUM_THREADS="2")
    san = subprocess.run([os.path.join(ORACLE, "rf_oracle_sanitized")], env=env, capture_output=True, text=True, timeout=600)
    assert san.returncode == 0, san.stderr[-4000:]
    assert "runtime error" not in san.stderr and "AddressSanitizer" not in san.stderr, san.stderr[-4000:]
    plain = subprocess.run([os.path.join(ORACLE, "rf_oracle_plain")], env=env, capture_output=True, text=True, timeout=600)
    assert plain.returncode == 0, plain.stderr[-4000:]
    assert len(san.stdout.strip()) == 16 and san.stdout == plain.stdout
