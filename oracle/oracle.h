/*
 * oracle.h -- CPU restatement of the reference CPU backend's kernel semantics.
 * Test infrastructure: see the header of oracle.c for what is restated and how
 * it is pinned.  Never part of the product path.
 */
#ifndef POLYGRAD_ORACLE_H
#define POLYGRAD_ORACLE_H

#include "polygrad_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Evaluates one scheduled kernel root on host buffers.  args[i] is the buffer of
 * PARAM i, followed by one pointer-to-int per DEFINE_VAR (src/exec_plan.c:1026-1041). */
int oracle_run_kernel(const PolyUOp *root, void **args, int n_args);

/* Evaluates a whole schedule: slot_data[i] must be a host buffer for every
 * external slot; intermediates are allocated (zero-filled) and freed here. */
int oracle_run_schedule(const PolySchedule *s, void **slot_data, int n_slots);

/* Scalar pieces, exposed so that tests can pin them one by one. */
float oracle_exp2f(float x);
double oracle_exp2(double x);
float oracle_log2f(float x);
double oracle_log2(double x);
uint64_t oracle_threefry(uint64_t x, uint64_t key);
uint16_t oracle_f32_to_bf16(float f);
float oracle_bf16_to_f32(uint16_t h);
uint16_t oracle_f32_to_f16(float f);
float oracle_f16_to_f32(uint16_t h);

#ifdef __cplusplus
}
#endif
#endif
