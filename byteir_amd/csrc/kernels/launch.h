// A kernel launch on `stream` without dynamic LDS; the kernel name goes in parentheses (its
// template arguments hold commas).  A host build of these sources for tests defines its own
// BRT_ROCM_LAUNCH before this header and runs the workgroups on the CPU.
#pragma once
#ifndef BRT_ROCM_LAUNCH
#define BRT_ROCM_LAUNCH(kernel, grid, block, stream, ...) kernel<<<(grid), (block), 0, (stream)>>>(__VA_ARGS__)
#endif
