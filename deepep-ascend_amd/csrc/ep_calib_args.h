// Kernel argument blocks of the calibration code object (ep_calib.hip), shared with its host side
// (ep_calib.cpp).  One struct by value per kernel, as in ep_args.h.
#pragma once
#include <stdint.h>

#include "ep_args.h"

// num_chunks chunks of 4 KiB starting at dst.
struct EpCalibFillArgs {
    void* dst;
    unsigned num_chunks;
    unsigned value;
    unsigned unit_chunks;         // scrambled order: consecutive chunks that stay together (a power of two)
    unsigned pad;                 // ep_calib_fill_affine: shift of the chunk inside its unit
};

// num_fronts fronts of rows: row n of front f starts at dst + f * front_pitch_bytes + n * row_bytes.
struct EpCalibFrontsArgs {
    void* dst;
    int64_t front_pitch_bytes;
    unsigned num_fronts, row_bytes;
    unsigned value, pad;
};

// Workgroup b writes chunk b of dst; reads_num of every reads_den workgroups also read a chunk of src.
struct EpCalibMixedArgs {
    const void* src;
    void* dst;
    unsigned num_read_chunks;
    unsigned reads_num, reads_den;
    unsigned value;
};

#ifdef __HIPCC__
typedef int2 ep_calib_entry_t;
#else
struct ep_calib_entry_t { int x, y; };
#endif

// Destination-ordered variants of the fused copy kernel.
struct EpCalibOrderedArgs {
    EpScatterArgs s;                  // inputs, outputs and padding geometry, as the product's copy kernel takes them
    const ep_calib_entry_t* order;    // [num_entries] (slot, token | position << 24); slot < 0: hole
    unsigned char* q_rows;            // two passes: [T, hidden] staged FP8 rows
    float* q_sf;                      // two passes: [T, hidden / 128] staged scales
    int num_entries;
    int groups;                       // wave tasks per entry
    int entries_per_list;             // steered: entries of one (chunk, XCD) list
    int wgs_per_list;                 // steered: workgroups serving one list
};
