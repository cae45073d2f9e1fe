// TEST INFRASTRUCTURE ONLY (see ratchet_cpu_oracle.h): function table exported by each build of orc_kernels.inc
#ifndef ORC_TABLE_H
#define ORC_TABLE_H
#include <stddef.h>
#include <stdint.h>
struct OrcTable {
    int (*binary)(int, int, const void*, const void*, void*, size_t);
    int (*unary)(int, int, const void*, void*, size_t);
    int (*cast)(int, int, const void*, void*, size_t);
    int (*permute)(int, const void*, void*, int, const uint64_t*, const uint32_t*);
    int (*slice)(int, const void*, void*, int, const uint64_t*, const uint64_t*, const uint64_t*);
    int (*broadcast)(int, const void*, void*, int, const uint64_t*, int, const uint64_t*, int);
    int (*concat)(int, int, const void* const*, int, const uint64_t*, int, void*);
    int (*cache)(int, void*, int, const uint64_t*, const void*, const uint64_t*, int, uint64_t, void*);
    int (*rope)(int, const void*, void*, const uint64_t*, uint64_t, float, uint64_t);
    int (*index_select)(int, const void*, int, const uint64_t*, const int32_t*, uint64_t, int, void*);
    int (*index_write)(int, void*, int, const uint64_t*, const void*, uint64_t, const uint64_t*);
    int (*softmax)(int, const void*, void*, size_t, size_t);
    int (*layer_norm)(int, const void*, const void*, const void*, void*, size_t, size_t, float, size_t);
    int (*rms_norm)(int, const void*, const void*, void*, size_t, size_t, float, size_t);
    int (*group_norm)(int, const void*, const void*, const void*, void*, size_t, size_t, size_t, size_t, float);
    size_t (*count_not_close)(int, const void*, const void*, size_t, double, double, double*);
    uint16_t (*f32_to_f16)(float);
    float (*f16_to_f32)(uint16_t);
    uint16_t (*f32_to_bf16)(float);
    float (*bf16_to_f32)(uint16_t);
};
namespace orc_soft { extern const OrcTable kTable; }
namespace orc_hw { extern const OrcTable kTable; }
#endif
