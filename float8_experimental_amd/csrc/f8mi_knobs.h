// Compile-time knobs for measurement builds of the library (python _build.py --out other.so -DF8MI_WALK_GROUP=2, loaded
// by pointing F8MI_LIB at the file).  The shipped library is built with the defaults below; every knob changes where
// and how bytes move, none changes a result.  f8mi_build_knobs() names the knobs a build was made with, so that a
// measurement build cannot pass for the shipped one.
#pragma once

// ---- tile walk of the 256 x 256-tile GEMM (f8mi_gemm_dma16_impl.h)
#ifndef F8MI_WALK_GROUP
#define F8MI_WALK_GROUP 4       // width of the bands the walk sweeps, in tiles
#endif
#ifndef F8MI_WALK_XCD_CHUNK
#define F8MI_WALK_XCD_CHUNK 0   // 0: each XCD owns one contiguous run of the tile order; n: chunks of n ids dealt round-robin
#endif
#ifndef F8MI_WALK_SHORT_SIDE
#define F8MI_WALK_SHORT_SIDE 0  // 1: sweep the bands along the shorter side of the tile grid
#endif
#ifndef F8MI_DMA_CACHE_POLICY   // cache-policy modifiers of the operand DMA (" nt", " sc1", ...)
#define F8MI_DMA_CACHE_POLICY ""
#define F8MI_DMA_CACHE_POLICY_IS_DEFAULT 1
#else
#define F8MI_DMA_CACHE_POLICY_IS_DEFAULT 0
#endif

// ---- cast kernel (f8mi_cast.hip)
#ifndef F8MI_CAST_REVERSE_WALK  // 1: last tiles first, the reverse of the order the amax pass read the tensor in
#define F8MI_CAST_REVERSE_WALK 0
#endif
#ifndef F8MI_CAST_NT_STORES     // 1: non-temporal stores of the fp8 bytes (16 % slower: 139 -> 161 us per launch in the
#define F8MI_CAST_NT_STORES 0   // benchmark step, alternated three times on one box)
#endif

// ---- amax kernel (f8mi_amax.hip): tensors of up to this many bytes are read with ordinary instead of non-temporal
// loads, which leave the tensor in the 256 MB memory-side cache for the cast that follows.  Measured in the benchmark
// step (kernel times from a trace, amax + cast of one tensor):
//   every tensor with ordinary loads: 134 MB 59.7 -> 55.7 us, 168 MB 72.5 -> 71.6, but 268 MB 111.6 -> 121.4,
//     470 MB 199.5 -> 238.4, 1.9 GB 774 -> 816 (the cast gains 3 - 10 %, the amax pass loses 30 - 70 %);
//   only tensors up to 192 MB with ordinary loads: 134 MB 59.7 -> 66.9 us, 168 MB 72.5 -> 80.9 -- worse than either.
// A line allocated in that cache pushes out a line that is there, and when that is a dirty line -- the fp8 copy or the
// GEMM output written just before -- its write-back competes with the reads: what ordinary loads cost depends on what
// the kernels before left in the cache, not on the tensor's size, and no size rule survives a change of neighbours.
#ifndef F8MI_AMAX_PLAIN_LOADS_MAX_BYTES
#define F8MI_AMAX_PLAIN_LOADS_MAX_BYTES 0
#endif
