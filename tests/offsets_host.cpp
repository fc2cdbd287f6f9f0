// Host-only check of the 32-bit weight-row offsets used when the forward resolves indices
// (mamtorch_amd/csrc/mam_offsets.h), at a weight matrix larger than 4 GiB that no GPU test allocates.
// Prints one line per failure and returns their number.
#include <stdio.h>

#include "../mamtorch_amd/csrc/mam_offsets.h"

static int check_set(int M, int ldw, int first, int rows_in_set)
{
    int bad = 0;
    const uint32_t ld_bytes = (uint32_t)ldw * 4u;
    const uint32_t last = mam::last_row_offset(M, first, rows_in_set, ld_bytes);
    for (int r = 0; r < rows_in_set; ++r) {
        const int neuron = (first + r) < M ? (first + r) : (M - 1);          // what the kernel must address
        const uint64_t want = (uint64_t)(neuron - first) * ld_bytes;           // exact, in 64 bits
        const uint32_t got = mam::clamped_row_offset((uint32_t)r * ld_bytes, last);
        if ((uint64_t)got != want) {
            printf("M=%d ldw=%d first=%d row %d: offset %u, want %llu\n", M, ldw, first, r, got,
                   (unsigned long long)want);
            ++bad;
        }
    }
    return bad;
}

int main()
{
    int bad = 0;
    // (M - 1) * ldw * 4 = 4295049216 wraps to 81920 in 32 bits: the first tile must not be clamped by it
    const int M = 262150, ldw = 4096;
    for (int first = 0; first < M; first += 64) bad += check_set(M, ldw, first, 64);
    for (int first = 0; first < M; first += 16) bad += check_set(M, ldw, first, 16);
    // a small ragged case
    for (int first = 0; first < 70; first += 64) bad += check_set(70, 128, first, 64);
    for (int first = 0; first < 70; first += 16) bad += check_set(70, 128, first, 16);
    printf("%d failures\n", bad);
    return bad ? 1 : 0;
}
