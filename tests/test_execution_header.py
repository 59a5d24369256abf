"""The header-only C++ scheduler mirror must compile as plain C++ against the C
ABI header (no HIP headers needed), and link against the library."""
import os
import subprocess
import tempfile

from conftest import ROOT

SRC = r"""
#include "cswap_execution.hpp"
#include <stdio.h>
int main() {
  cswap::Execution exe(nullptr);
  exe.init_(45);
  exe.policy[2] = 3; exe.policy[6] = 6;
  exe.preforward();
  int rc = exe.pre(-1, nullptr, 1, 1, 1, nullptr);       // untracked input: nothing happens
  int id = exe.post();
  rc |= exe.pre(0, nullptr, 1, 1, 1, nullptr);            // policy 0: kept
  exe.post();
  std::vector<cswap::Execution::Input> two = {{0, nullptr, 1, 1, 1}, {-1, nullptr, 1, 1, 1}};
  rc |= exe.pre(two, nullptr, cswap::CONV);               // an op with two inputs, neither swapped
  int id2 = exe.post();
  rc |= (exe.prefetch(7) == CSWAP_E_STATE) ? 0 : 1;       // nothing was swapped under id 7
  exe.postforward();
  printf("%d %d %d %d %d\n", rc, id, id2, exe.index, (int)exe.swapped(0));
  return (rc == 0 && id == 0 && id2 == 2 && exe.index == 2 && !exe.swapped(0) && exe.com_and_tran(5) == 0) ? 0 : 1;
}
"""


def test_header_compiles_links_and_schedules():
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.cpp")
        exe = os.path.join(d, "t")
        open(src, "w").write(SRC)
        lib = os.path.join(ROOT, "cswap_amd", "libcswap_hip.so")
        subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), src, lib,
                               "-Wl,-rpath," + os.path.dirname(lib), "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib",
                               "-lamdhip64", "-o", exe])
        subprocess.check_call([exe])


BRANCHES = r"""
#include "cswap_execution.hpp"
#include <stdio.h>
using cswap::Execution;
int main() {
  // Execution.h:70,86,107,243 as a table: entry of policy[], global mode, consumer -> action
  struct Row { int entry, mode, layer, want; };
  const Row rows[] = {
    {0, 1, cswap::ACT, 0},  {0, 1, cswap::CONV, 0}, {2, 1, cswap::ACT, 2},  {3, 1, cswap::CONV, 3},
    {6, 1, cswap::POOL, 6}, {-1, 1, cswap::BN, -1}, {1, 1, cswap::CONV, 1}, {1, 3, cswap::CONV, 1},
    {0, 3, cswap::CONV, 2}, {3, 3, cswap::CONV, 2}, {6, 4, cswap::CONV, 2}, {0, 3, cswap::ACT, 0},
    {3, 3, cswap::POOL, 3}, {0, 4, cswap::ACT, 1},  {2, 4, cswap::BN, 1},   {6, 4, cswap::FC, 1},
    {0, 2, cswap::CONV, 0}, {2, 2, cswap::CONV, 2}, {5, 1, cswap::ACT, 0},
  };
  for (const Row& r : rows)
    if (Execution::action(r.entry, r.mode, (cswap::Layer_type)r.layer) != r.want) {
      printf("entry %d mode %d layer %d: got %d want %d\n", r.entry, r.mode, r.layer,
             Execution::action(r.entry, r.mode, (cswap::Layer_type)r.layer), r.want);
      return 1;
    }
  // dropped tensors never reach the engine: tag 1 until the next iteration starts
  Execution exe(nullptr);
  exe.init_(8);
  exe.policy[0] = 1;
  exe.policy_ = 4;                       // SuperNeurons: everything that does not feed a convolution is dropped
  exe.preforward();
  exe.pre(-1, nullptr, 1, 1, 1, nullptr, cswap::CONV); exe.post();        // op 0
  if (exe.pre(0, nullptr, 4, 4, 4, nullptr, cswap::CONV)) return 2;       // op 1 consumes tensor 0: policy 1 -> drop
  exe.post();
  if (exe.pre(1, nullptr, 4, 4, 4, nullptr, cswap::ACT)) return 3;        // op 2 consumes tensor 1: mode 4, not CONV
  exe.post();
  if (exe.com_and_tran(0) != 1 || exe.com_and_tran(1) != 1 || !exe.dropped(1) || exe.swapped(1)) return 4;
  float dummy;
  if (exe.fetch(1, &dummy, nullptr) != CSWAP_E_STATE) return 5;           // nothing to bring back: recompute
  exe.preforward();
  if (exe.com_and_tran(0) != 0 || exe.dropped(1)) return 6;
  return 0;
}
"""

CALL_SITE = r"""
#include "cswap_compat.h"
struct Tensor { void* p; long n; void* data_ptr() const { return p; } long numel() const { return n; } };
void* buffer;
size_t buffersize;
void at_the_call_site(Tensor& pre)
{
  buffer = compress(pre.data_ptr(), pre.numel(), buffersize);   // CSWAP+/Execution.h:113, verbatim
  setRatio(128);                                                // CSWAP+/Execution.h:63
}
int main() { return 0; }
"""


def _build_and_run(source, name):
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, name + ".cpp")
        exe = os.path.join(d, name)
        open(src, "w").write(source)
        lib = os.path.join(ROOT, "cswap_amd", "libcswap_hip.so")
        subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), src, lib,
                               "-Wl,-rpath," + os.path.dirname(lib), "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib",
                               "-lamdhip64", "-o", exe])
        subprocess.check_call([exe])


def test_branch_table_of_the_reference_scheduler():
    """policy[] entries 0/1/2/3/6, the global modes policy_ 1-4 and the consumer's
    layer type combine as in the reference (Execution.h:70,86,107,243)."""
    _build_and_run(BRANCHES, "branches")


def test_python_mirror_has_the_same_branch_table():
    from cswap_amd.execution import ACT, BN, CONV, FC, POOL, Execution

    rows = [(0, 1, ACT, 0), (0, 1, CONV, 0), (2, 1, ACT, 2), (3, 1, CONV, 3), (6, 1, POOL, 6), (-1, 1, BN, -1),
            (1, 1, CONV, 1), (1, 3, CONV, 1), (0, 3, CONV, 2), (3, 3, CONV, 2), (6, 4, CONV, 2), (0, 3, ACT, 0),
            (3, 3, POOL, 3), (0, 4, ACT, 1), (2, 4, BN, 1), (6, 4, FC, 1), (0, 2, CONV, 0), (2, 2, CONV, 2),
            (5, 1, ACT, 0)]
    for entry, mode, layer, want in rows:
        assert Execution.action(entry, mode, layer) == want, (entry, mode, layer)


def test_the_reference_call_form_of_compress_compiles_unchanged():
    _build_and_run(CALL_SITE, "call_site")
