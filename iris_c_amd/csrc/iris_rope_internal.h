/*
 * Shared between the host table builders (iris_rope_tables.c) and the device
 * entries (iris_rocm.c), so that both take their column frequencies and
 * positions from the same code. Not part of the public interface.
 */
#ifndef IRIS_ROPE_INTERNAL_H
#define IRIS_ROPE_INTERNAL_H

#include <stddef.h>
#include <stdint.h>

/* A table as a dictionary of its distinct (axis, position) rows plus one offset per (row, axis);
 * see iris_rope_tables.c. values and index are malloc'd. */
int iris_rope_dictionary_(const void *pos, int use_double, int seq, int naxes, const int *axis_dims,
                          const int *axis_lens, float theta, float **values, size_t *n_values, uint32_t **index);
/* malloc'd positions of the text encoder's rows, NULL on failure */
int *iris_rope_qwen3_positions_(const int *attention_mask, int seq, int pad_at_one);
/* argument check of the expansion routines: 1 = usable */
int iris_rope_axes_ok_(int seq, int naxes, const int *axis_dims);

#endif
