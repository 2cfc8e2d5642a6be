// Host-side simplification of the batch shape before launch.
#pragma once

#include <stdint.h>

#include "km_common.h"

namespace km {

// Drops batch dimensions of size 1 and merges adjacent dimensions that every tensor walks
// with one stride (stride[d] == stride[d+1] * size[d+1], which includes two broadcast
// dimensions of stride 0).  The flat batch index keeps its meaning, so outputs laid out
// contiguously over the original batch shape are unaffected.  After this most calls have
// batch rank 0 or 1 and the per-wavefront index arithmetic on the device is trivial.
template <int NT>
inline void collapse_batch(int rank, const int64_t* sizes, const int64_t* const (&strides)[NT],
                           BatchShape* shape, BatchStrides* (&out)[NT]) {
    int64_t csize[KM_MAX_BATCH_RANK];
    int64_t cstride[NT][KM_MAX_BATCH_RANK];
    int crank = 0;
    for (int d = 0; d < rank; d++) {
        if (sizes[d] == 1) {
            continue;
        }
        bool merge = crank > 0;
        if (merge) {
            for (int t = 0; t < NT; t++) {
                if (cstride[t][crank - 1] != strides[t][d] * sizes[d]) {
                    merge = false;
                    break;
                }
            }
        }
        if (merge) {
            csize[crank - 1] *= sizes[d];
            for (int t = 0; t < NT; t++) {
                cstride[t][crank - 1] = strides[t][d];
            }
        } else {
            csize[crank] = sizes[d];
            for (int t = 0; t < NT; t++) {
                cstride[t][crank] = strides[t][d];
            }
            crank++;
        }
    }
    shape->rank = crank;
    for (int d = 0; d < KM_MAX_BATCH_RANK; d++) {
        shape->sizes[d] = d < crank ? (int)csize[d] : 1;
        for (int t = 0; t < NT; t++) {
            out[t]->s[d] = d < crank ? cstride[t][d] : 0;
        }
    }
}

}  // namespace km
