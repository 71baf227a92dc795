// File input of the clusterNet host API: read_hdf5 of source/util.cu:100-131, without libhdf5.
//
// The reference's data files (tests/*.hdf5, source/8bit_floats.hdf5) are what h5py writes for a plain
// array: superblock version 0, one old-style group (B-tree + local heap), version 1 object headers and
// a contiguous, unfiltered dataset.  The reader below understands exactly that subset and refuses
// anything else (chunked or compressed layouts, new-style groups, big-endian or compound types) with
// a message.  Like the reference's H5Dread with H5T_NATIVE_FLOAT, it converts float64 and integer
// datasets to fp32.
#ifndef CLUSTERNET_FACADE_UTIL_H
#define CLUSTERNET_FACADE_UTIL_H

#include "basicOps.h"

// Host matrix (free with free_cpu_matrix) holding dataset "/Default" (or `tag`, with or without the
// leading slash) of the file.  One-dimensional datasets come back as n x 1.  Throws a const char *.
Matrix *read_hdf5(const char *filepath);
Matrix *read_hdf5(const char *filepath, const char *tag);

extern "C" {
// C entry for bindings: 0 on success; on failure returns non-zero and *error_text points to a static
// message.  *data is malloc'd (rows * cols floats) and owned by the caller.
int cn_facade_read_hdf5(const char *filepath, const char *tag, long long *rows, long long *cols, float **data,
                        const char **error_text);
}

#endif
