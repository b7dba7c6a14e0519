// The planned form of a tile-pruned linear (what et_tile_plan_create builds and
// Linear_tile owns), shared by the linear kernels and the layer-tail kernel.
#pragma once
#include "common.h"

#include <vector>

namespace et {
struct TailProgram;
void tail_program_destroy(TailProgram *p);
} // namespace et

struct et_tile_plan {
    int in_feat = 0, out_feat = 0, ntile = 0, KC = 0, nchunk = 0;
    et::f16 *d_data = nullptr;
    int *d_cptr = nullptr;
    int *d_row_offset = nullptr;
    et::f16 *d_bias = nullptr;
    // Host copy of the caller's tile_mat with every block-row's tiles sorted by
    // column: the layer-tail program (tile_tail.hip) is built from it.
    std::vector<int> h_row_ptr, h_col;
    std::vector<uint16_t> h_data;
    unsigned long long uid = 0; // never reused: identifies a plan beyond its address
    // Second feed-forward linear only: the layer-tail program built for it
    // together with the projection and first feed-forward plans tail_uid names.
    et::TailProgram *tail = nullptr;
    unsigned long long tail_uid[2] = {0, 0};
};

namespace et {
// One int per process in pinned host memory that kernels set when a bounded
// wait inside a workgroup gives up (device pointer / host pointer, null if the
// allocation failed).  The launchers of those kernels read it before every
// launch and report ET_ERR_HIP once.
int *wait_status_device();
volatile int *wait_status_host();
int check_wait_status(const char *who);

// layer tail as pairs of workgroups over 64-row panels (tile_tail.hip)
size_t tail_ws_bytes_for(int D, int rows);
size_t tail_pair_ws_bytes(const et_tile_plan *pO, const et_tile_plan *p1, const et_tile_plan *p2, int M);
int tail_pair_prepare(const et_tile_plan *pO, const et_tile_plan *p1, et_tile_plan *p2);
bool tail_pair_forced();
bool tail_pair_enabled();
bool tail_pair_applies(const et_tile_plan *pO, const et_tile_plan *p1, const et_tile_plan *p2);
int tail_pair_launch(const et_tile_plan *pO, const et_tile_plan *p1, const et_tile_plan *p2, f16 *Y,
                     const f16 *attn, const f16 *input, const f16 *gamma1, const f16 *beta1,
                     const f16 *gamma2, const f16 *beta2, int M, void *ws, hipStream_t st);
} // namespace et
