/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the Hawk RG-LRU hot path (scan forward / backward, temporal conv1d,
 * decode steps) in plain C.  Only tests, the smoke check and the benchmark's cpu_baseline
 * leg may load this library; the product path never does.
 *
 * The restatement follows hawk/scan_fused.py, hawk/external.py, hawk/cache.py and
 * hawk/hawk.py of the upstream tree line by line in meaning (citations sit on each
 * function in rglru_oracle_impl.h) but evaluates everything in the working precision with
 * no bf16 rounding of stores, so the _f64 build is the ground truth the parity
 * tolerances are measured against.
 *
 * How each function is pinned (upstream holds no tests or golden vectors):
 *   scan fwd   constant-gate case equals scipy.signal.lfilter; r -> 0 gives h == 0;
 *              agreement with an independent torch loop over the one-token decode step.
 *   scan bwd   agreement with torch.autograd through that torch loop (clipped sqrt
 *              derivative included), finite differences away from the clip, and the
 *              closed form csg == 1000 inside the clip.
 *   conv       torch.nn.functional.conv1d (depthwise, left pad W-1) and its autograd.
 *   steps      prefill(T) + step == scan / conv over T+1 rows.
 */
#include <math.h>
#include <stddef.h>

#define REAL double
#define SUFFIX _f64
#include "rglru_oracle_impl.h"
#undef REAL
#undef SUFFIX

#define REAL float
#define SUFFIX _f32
#include "rglru_oracle_impl.h"
#undef REAL
#undef SUFFIX
