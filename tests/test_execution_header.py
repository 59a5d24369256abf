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
