// Compile-time helpers for software-pipelined loops on gfx950.
//
// Why they exist: when a load of a loop sits behind a branch (a per-lane condition, or "is there a next
// item"), the compiler no longer knows how many loads are outstanding at a use and waits for all of
// them, so nothing stays in flight across iterations. Here every step of a pipeline is compiled knowing
// how many items follow it, and register sets rotate by unrolling instead of by copies.
#pragma once
#include <type_traits>

template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

// A software pipeline over `count` items with SETS rotating register sets. step(set, rem, i) works on
// item i with register set `set` (std::integral_constant) and is told, as a compile-time constant `rem`
// capped at NEED, how many items follow it: so what a step still requests (items i + 1 .. i + NEED) is
// decided when it is compiled, no load of the loop sits behind a branch, the compiler can count exactly
// which loads a use waits for, and the later ones stay in flight. The loop runs rounds of SETS steps
// while every step of a round has NEED followers; the last items run as one straight-line sequence
// chosen by how many are left. NEED >= SETS - 1.
template <int SETS, int NEED, int R, int J = 0, typename Step>
__device__ __forceinline__ void pipeline_last(Step& step, int i) {
  if constexpr (J < R) {
    step(std::integral_constant<int, J % SETS>{}, std::integral_constant<int, (R - J - 1 < NEED ? R - J - 1 : NEED)>{},
         i + J);
    pipeline_last<SETS, NEED, R, J + 1>(step, i);
  }
}
template <int SETS, int NEED, int R = 1, typename Step>
__device__ __forceinline__ void pipeline_last_of(Step& step, int i, int left) {
  if constexpr (R < SETS + NEED) {
    if (left == R)
      pipeline_last<SETS, NEED, R>(step, i);
    else
      pipeline_last_of<SETS, NEED, R + 1>(step, i, left);
  }
}
template <int SETS, int NEED, int S = 0, typename Step>
__device__ __forceinline__ void pipeline_round(Step& step, int i) {
  if constexpr (S < SETS) {
    step(std::integral_constant<int, S>{}, std::integral_constant<int, NEED>{}, i + S);
    pipeline_round<SETS, NEED, S + 1>(step, i);
  }
}
template <int SETS, int NEED, typename Step>
__device__ __forceinline__ void run_pipeline(Step& step, int count) {
  static_assert(NEED >= SETS - 1 && NEED >= 1, "a step must know about every item it may request");
  int i = 0;
  for (; i + SETS + NEED <= count; i += SETS) pipeline_round<SETS, NEED>(step, i);
  pipeline_last_of<SETS, NEED>(step, i, count - i);
}
