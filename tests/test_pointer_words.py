"""Host check of the address re-assembly used by the LDS-DMA helper of the latent decode kernel
(tt-xla_amd/csrc/pointer_words.h, used by dma16_uniform in common.h): the two 32-bit words of a
device address come back from a lane broadcast as signed ints, and a low word with bit 31 set
must not leak into the high word.  The header is plain C++: it is compiled with g++ and run here."""

import os
import subprocess
import textwrap

import __graft_entry__ as entry

CSRC = os.path.join(entry.PKG_ROOT, "csrc")

PROGRAM = textwrap.dedent(
    r"""
    #include <stdio.h>
    #include "pointer_words.h"
    int main() {
      const uint64_t cases[] = {
          0x00007f3a80001000ull,  // low word with bit 31 set: the case that faulted
          0x00007f3affffffe0ull, 0x00007f3a7ffffff0ull, 0x0000000080000000ull,
          0x00007fff00000000ull, 0xffffffffffffffffull, 0x0000000000000010ull,
          0x8000000080000000ull,
      };
      int bad = 0;
      for (uint64_t a : cases) {
        const int lo = (int)(uint32_t)a, hi = (int)(uint32_t)(a >> 32);  // what the broadcast returns
        const uint64_t got = ttpa::address_from_words(lo, hi);
        if (got != a) { printf("MISMATCH %016llx -> %016llx\n", (unsigned long long)a, (unsigned long long)got); bad = 1; }
        // the defect: widening the signed low word
        const uint64_t wrong = ((uint64_t)(uint32_t)hi << 32) | (uint64_t)(int64_t)lo;
        if (((uint32_t)a & 0x80000000u) && (uint32_t)(a >> 32) != 0xffffffffu) { if (wrong == a) { printf("sign extension not visible for %016llx\n", (unsigned long long)a); bad = 1; } }
      }
      printf(bad ? "FAIL\n" : "OK\n");
      return bad;
    }
    """
)


def test_address_from_words(tmp_path):
    src = tmp_path / "words.cc"
    src.write_text(PROGRAM)
    exe = tmp_path / "words"
    subprocess.run(["g++", "-std=c++17", "-O1", "-I", CSRC, str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip().endswith("OK"), out.stdout + out.stderr
