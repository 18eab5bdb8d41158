// Single-launch decode step for one token, sharded over the eight compute dies of the GPU (decode_die.hip).
#pragma once

#include "stage.hpp"

namespace mesh {

struct DieDecode;      // per-session state: exchange buffers, barrier counters, the per-layer weight table

// Whether the stage has the shape this kernel is built for (see decode_die.hip) and the device its geometry.
bool die_decode_eligible(const mesh_stage *st);
// Allocates the state for `s`; *out stays null (and MESH_OK is returned) when the stage is not eligible or the placement
// probe shows that workgroups do not land on the dies the kernel assumes.
int die_decode_create(mesh_session *s, DieDecode **out);
void die_decode_destroy(DieDecode *d);
// All layers of the stage for the one token whose position / sequence are in s->d_pos / s->d_seq: s->x in, s->x out.
int die_decode_step(mesh_session *s, DieDecode *d);
// After the stream has been synchronised: MESH_ERR_DEVICE if a wait inside the kernel gave up (the step's output is then
// undefined); the state is reset so that later steps can run.
int die_decode_check(mesh_session *s, DieDecode *d);

}  // namespace mesh
