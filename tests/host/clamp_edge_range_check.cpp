// Host-side check of the arithmetic that keeps a node's edge range inside the edge arrays (cm::clamp_edge_range):
// compiled for the host only and run by tests/test_cabi_host.py.  Prints "ok" on success.
#include <cstdio>
#include <cstdlib>

#include "common.hpp"

static void expect(int e0, int e1, long long nedges, int want0, int want1) {
  cm::clamp_edge_range(e0, e1, nedges);
  if (e0 != want0 || e1 != want1) {
    std::printf("clamp_edge_range gave [%d, %d), expected [%d, %d)\n", e0, e1, want0, want1);
    std::exit(1);
  }
}

int main() {
  expect(3, 9, 20, 3, 9);              // a valid range is left alone
  expect(0, 20, 20, 0, 20);
  expect(7, 7, 20, 7, 7);              // empty
  expect(-5, 4, 20, 0, 4);             // start below the arrays
  expect(2, 99, 20, 2, 20);            // end beyond the arrays
  expect(12, 5, 20, 12, 12);           // reversed (unsorted list): empty, not negative
  expect(50, 60, 20, 20, 20);          // both beyond
  expect(-9, -2, 20, 0, 0);            // both below
  expect(1 << 30, -(1 << 30), 0, 0, 0);  // no edges at all
  // every range of garbage offsets ends up inside [0, nedges] with e0 <= e1
  unsigned state = 12345u;
  for (int it = 0; it < 100000; ++it) {
    state = state * 1664525u + 1013904223u;
    int a = static_cast<int>(state);
    state = state * 1664525u + 1013904223u;
    int b = static_cast<int>(state);
    const long long ne = (state >> 7) % 1000;
    cm::clamp_edge_range(a, b, ne);
    if (a < 0 || b < a || b > ne) {
      std::printf("range [%d, %d) escapes [0, %lld]\n", a, b, ne);
      return 1;
    }
  }
  std::printf("ok\n");
  return 0;
}
