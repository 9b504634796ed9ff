// ArgMax of a pooling window with the native backend's reduction order (CX/native/reduce.h:46-83, as ArgMax over the kernel axes of
// the Im2Col'ed windows runs through it, CX/native/native_device/pool.cc:97-113): elements are taken four at a time as a small
// tree, the groups of a 32-element block accumulate left to right, blocks are merged pairwise, the tail that does not fill a group
// of four comes last.  A later element replaces the current best only when it is strictly larger, so ties go to the element the
// order meets first and a NaN neither replaces nor is replaced.  Shared by the 2-D pooling gradients and the n-axis ones.
#pragma once

#include "common.h"

namespace hipcx {

template <typename V>
struct WinBest {
    V v;
    int i;  // < 0: empty
};

template <typename V>
__device__ __forceinline__ void WinReduce(WinBest<V> next, WinBest<V>& acc) {  // ArgMax's rule: a later element must be strictly larger
    if (next.i < 0) return;
    if (acc.i < 0 || acc.v < next.v) acc = next;
}

// Comparison type of a window's elements: float16 compares as float, bool as int.
template <typename T>
using win_value_t = std::conditional_t<std::is_same<T, half_t>::value, float, std::conditional_t<std::is_same<T, bool>::value, int, T>>;

// Index of the maximum of fetch(0) .. fetch(len - 1) in that order; fetch is called once per index, in ascending order.
template <typename V, typename Fetch>
__device__ __forceinline__ int NativeOrderArgMax(int len, Fetch&& fetch) {
    using B = WinBest<V>;
    int i = 0;
    auto next_elem = [&]() -> B {
        B b{fetch(i), i};
        ++i;
        return b;
    };
    const int main_len = len - (len % 4);
    B accum{V(0), -1};
    if (main_len <= 32) {  // one block of the tree: groups of four, then the tail (every usual window)
        while (i < main_len) {
            B p0 = next_elem();
            WinReduce(next_elem(), p0);
            B p1 = next_elem();
            WinReduce(next_elem(), p1);
            WinReduce(p1, p0);
            WinReduce(p0, accum);
        }
        while (i < len) WinReduce(next_elem(), accum);
        return accum.i;
    }
    B tree[26];
    while (i < main_len) {
        if (i != 0 && i % 32 == 0) {
            int lvl = 0;
            for (int k = i >> 1; k % 32 == 0; k >>= 1, ++lvl) WinReduce(tree[lvl], accum);
            tree[lvl] = accum;
            accum = B{V(0), -1};
        }
        B p0 = next_elem();
        WinReduce(next_elem(), p0);
        B p1 = next_elem();
        WinReduce(next_elem(), p1);
        WinReduce(p1, p0);
        WinReduce(p0, accum);
    }
    while (i < len) WinReduce(next_elem(), accum);
    int lvl = 0;
    for (int k = (len / 4 - 1) / 8; k > 0; k >>= 1, ++lvl) {
        if (k & 1) WinReduce(tree[lvl], accum);
    }
    return accum.i;
}

}  // namespace hipcx
