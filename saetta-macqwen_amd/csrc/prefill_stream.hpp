// The instruction streams of the prefill attention kernel's inner loop (hand-scheduled MFMAs, LDS fragment reads
// and global -> LDS copies), in a file of their own so that the calibration kernel of bench.py runs the very same
// streams.  Included inside a namespace that has the vector typedefs half8 (8 x _Float16) and floatx16 (16 x float).

// What a wave copies global -> LDS per step: 8 KB as eight global_load_lds_dwordx4 (64 lanes x
// 16 bytes each).  Inside the MFMA stream they are spread between the MFMAs, so that the
// texture path drains between them and their issue never stalls the wave.
struct Copy {
    uint64_t src;  // global address of the 8 KB (wave-uniform)
    uint32_t dst;  // LDS byte address they go to (wave-uniform)
};

__device__ __forceinline__ void copy_plain(const Copy &c, uint32_t lane16) {
    asm volatile(
        "s_mov_b32 m0, %[dst]\n"
        "s_nop 0\n"
        "global_load_lds_dwordx4 %[off], %[src]\n"
        "global_load_lds_dwordx4 %[off], %[src] offset:1024\n"
        "global_load_lds_dwordx4 %[off], %[src] offset:2048\n"
        "global_load_lds_dwordx4 %[off], %[src] offset:3072\n"
        "s_add_u32 m0, m0, 0x1000\n"
        "s_nop 0\n"
        "global_load_lds_dwordx4 %[off], %[src2]\n"
        "global_load_lds_dwordx4 %[off], %[src2] offset:1024\n"
        "global_load_lds_dwordx4 %[off], %[src2] offset:2048\n"
        "global_load_lds_dwordx4 %[off], %[src2] offset:3072\n"
        :
        : [off] "v"(lane16), [src] "s"(c.src), [src2] "s"(c.src + 4096), [dst] "s"(c.dst)
        : "memory", "m0");
}

// S^T = K Q^T of one block as one instruction stream: 16 LDS reads of K fragments kept four
// ahead of the 16 MFMAs that use them.  kaddr: LDS byte address of the K part plus 16 lane.
// Ends with the wait states an MFMA result needs before vector ALU instructions may read it.
// (Used before the loop only; in the loop the scores are part of stream_block.)
__device__ __forceinline__ void scores_block(floatx16 &s, const half8 (&q)[16], uint32_t kaddr) {
    half8 a0, a1, a2, a3;
#define SAETTA_S_STEP(A, Q, OFF, CNT)                                  \
    "s_waitcnt lgkmcnt(" #CNT ")\n"                                    \
    "v_mfma_f32_32x32x16_f16 %[s], %[" #A "], %[" #Q "], %[s]\n"       \
    "ds_read_b128 %[" #A "], %[addr] offset:" #OFF "\n"
#define SAETTA_S_LAST(A, Q, CNT)                                       \
    "s_waitcnt lgkmcnt(" #CNT ")\n"                                    \
    "v_mfma_f32_32x32x16_f16 %[s], %[" #A "], %[" #Q "], %[s]\n"
    asm volatile(
        "s_waitcnt lgkmcnt(0)\n"
        "ds_read_b128 %[a0], %[addr]\n"
        "ds_read_b128 %[a1], %[addr] offset:1024\n"
        "ds_read_b128 %[a2], %[addr] offset:2048\n"
        "ds_read_b128 %[a3], %[addr] offset:3072\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q0], 0\n"
        "ds_read_b128 %[a0], %[addr] offset:4096\n"
        SAETTA_S_STEP(a1, q1, 5120, 3) SAETTA_S_STEP(a2, q2, 6144, 3) SAETTA_S_STEP(a3, q3, 7168, 3)
        SAETTA_S_STEP(a0, q4, 8192, 3) SAETTA_S_STEP(a1, q5, 9216, 3) SAETTA_S_STEP(a2, q6, 10240, 3)
        SAETTA_S_STEP(a3, q7, 11264, 3) SAETTA_S_STEP(a0, q8, 12288, 3) SAETTA_S_STEP(a1, q9, 13312, 3)
        SAETTA_S_STEP(a2, q10, 14336, 3) SAETTA_S_STEP(a3, q11, 15360, 3)
        SAETTA_S_LAST(a0, q12, 3) SAETTA_S_LAST(a1, q13, 2) SAETTA_S_LAST(a2, q14, 1) SAETTA_S_LAST(a3, q15, 0)
        "s_nop 15\n"
        "s_nop 3\n"
        : [s] "=&v"(s), [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3)
        : [addr] "v"(kaddr), [q0] "v"(q[0]), [q1] "v"(q[1]), [q2] "v"(q[2]), [q3] "v"(q[3]), [q4] "v"(q[4]),
          [q5] "v"(q[5]), [q6] "v"(q[6]), [q7] "v"(q[7]), [q8] "v"(q[8]), [q9] "v"(q[9]), [q10] "v"(q[10]),
          [q11] "v"(q[11]), [q12] "v"(q[12]), [q13] "v"(q[13]), [q14] "v"(q[14]), [q15] "v"(q[15])
        : "memory");
#undef SAETTA_S_STEP
#undef SAETTA_S_LAST
}

// One step of a wave as one instruction stream: O^T += V^T P^T of the block whose
// probabilities are in p, interleaved MFMA by MFMA with S^T = K Q^T of the wave's next block
// (the scores chain through one accumulator, so alone they would wait on each other), 32 LDS
// fragment reads kept four ahead of the MFMAs, and the wave's copy.  kaddr / vaddr: LDS byte
// addresses of the next block's K part / this block's V^T part, plus 16 lane.  V^T fragment
// 2 mt + sp serves accumulator mt with k-step sp.  Ends with the wait states an MFMA result
// needs before vector ALU instructions may read it.
__device__ __forceinline__ void stream_block(floatx16 &s, floatx16 (&o)[8], const half8 (&q)[16], const half8 (&p)[2],
                                             uint32_t kaddr, uint32_t vaddr, const Copy &c, uint32_t lane16) {
    half8 a0, a1, a2, a3;
    asm volatile(
        "s_waitcnt lgkmcnt(0)\n"
        "s_mov_b32 m0, %[dst]\n"
        "ds_read_b128 %[a0], %[kaddr] offset:0\n"
        "ds_read_b128 %[a1], %[vaddr] offset:0\n"
        "ds_read_b128 %[a2], %[kaddr] offset:1024\n"
        "ds_read_b128 %[a3], %[vaddr] offset:2048\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q0], 0\n"
        "ds_read_b128 %[a0], %[kaddr] offset:2048\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o0], %[a1], %[p0], %[o0]\n"
        "ds_read_b128 %[a1], %[vaddr] offset:4096\n"
        "global_load_lds_dwordx4 %[off], %[src] offset:0\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a2], %[q1], %[s]\n"
        "ds_read_b128 %[a2], %[kaddr] offset:3072\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o1], %[a3], %[p0], %[o1]\n"
        "ds_read_b128 %[a3], %[vaddr] offset:6144\n"
        "global_load_lds_dwordx4 %[off], %[src] offset:1024\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q2], %[s]\n"
        "ds_read_b128 %[a0], %[kaddr] offset:4096\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o2], %[a1], %[p0], %[o2]\n"
        "ds_read_b128 %[a1], %[vaddr] offset:8192\n"
        "global_load_lds_dwordx4 %[off], %[src] offset:2048\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a2], %[q3], %[s]\n"
        "ds_read_b128 %[a2], %[kaddr] offset:5120\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o3], %[a3], %[p0], %[o3]\n"
        "ds_read_b128 %[a3], %[vaddr] offset:10240\n"
        "global_load_lds_dwordx4 %[off], %[src] offset:3072\n"
        "s_add_u32 m0, m0, 0x1000\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q4], %[s]\n"
        "ds_read_b128 %[a0], %[kaddr] offset:6144\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o4], %[a1], %[p0], %[o4]\n"
        "ds_read_b128 %[a1], %[vaddr] offset:12288\n"
        "global_load_lds_dwordx4 %[off], %[src2] offset:0\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a2], %[q5], %[s]\n"
        "ds_read_b128 %[a2], %[kaddr] offset:7168\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o5], %[a3], %[p0], %[o5]\n"
        "ds_read_b128 %[a3], %[vaddr] offset:14336\n"
        "global_load_lds_dwordx4 %[off], %[src2] offset:1024\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q6], %[s]\n"
        "ds_read_b128 %[a0], %[kaddr] offset:8192\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o6], %[a1], %[p0], %[o6]\n"
        "ds_read_b128 %[a1], %[vaddr] offset:1024\n"
        "global_load_lds_dwordx4 %[off], %[src2] offset:2048\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a2], %[q7], %[s]\n"
        "ds_read_b128 %[a2], %[kaddr] offset:9216\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o7], %[a3], %[p0], %[o7]\n"
        "ds_read_b128 %[a3], %[vaddr] offset:3072\n"
        "global_load_lds_dwordx4 %[off], %[src2] offset:3072\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q8], %[s]\n"
        "ds_read_b128 %[a0], %[kaddr] offset:10240\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o0], %[a1], %[p1], %[o0]\n"
        "ds_read_b128 %[a1], %[vaddr] offset:5120\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a2], %[q9], %[s]\n"
        "ds_read_b128 %[a2], %[kaddr] offset:11264\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o1], %[a3], %[p1], %[o1]\n"
        "ds_read_b128 %[a3], %[vaddr] offset:7168\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q10], %[s]\n"
        "ds_read_b128 %[a0], %[kaddr] offset:12288\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o2], %[a1], %[p1], %[o2]\n"
        "ds_read_b128 %[a1], %[vaddr] offset:9216\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a2], %[q11], %[s]\n"
        "ds_read_b128 %[a2], %[kaddr] offset:13312\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o3], %[a3], %[p1], %[o3]\n"
        "ds_read_b128 %[a3], %[vaddr] offset:11264\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q12], %[s]\n"
        "ds_read_b128 %[a0], %[kaddr] offset:14336\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o4], %[a1], %[p1], %[o4]\n"
        "ds_read_b128 %[a1], %[vaddr] offset:13312\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a2], %[q13], %[s]\n"
        "ds_read_b128 %[a2], %[kaddr] offset:15360\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[o5], %[a3], %[p1], %[o5]\n"
        "ds_read_b128 %[a3], %[vaddr] offset:15360\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q14], %[s]\n"
        "s_waitcnt lgkmcnt(2)\n"
        "v_mfma_f32_32x32x16_f16 %[o6], %[a1], %[p1], %[o6]\n"
        "s_waitcnt lgkmcnt(1)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a2], %[q15], %[s]\n"
        "s_waitcnt lgkmcnt(0)\n"
        "v_mfma_f32_32x32x16_f16 %[o7], %[a3], %[p1], %[o7]\n"
        "s_nop 15\n"
        "s_nop 3\n"
        : [s] "=&v"(s), [o0] "+v"(o[0]), [o1] "+v"(o[1]), [o2] "+v"(o[2]), [o3] "+v"(o[3]), [o4] "+v"(o[4]),
          [o5] "+v"(o[5]), [o6] "+v"(o[6]), [o7] "+v"(o[7]), [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2),
          [a3] "=&v"(a3)
        : [kaddr] "v"(kaddr), [vaddr] "v"(vaddr), [q0] "v"(q[0]), [q1] "v"(q[1]), [q2] "v"(q[2]), [q3] "v"(q[3]),
          [q4] "v"(q[4]), [q5] "v"(q[5]), [q6] "v"(q[6]), [q7] "v"(q[7]), [q8] "v"(q[8]), [q9] "v"(q[9]),
          [q10] "v"(q[10]), [q11] "v"(q[11]), [q12] "v"(q[12]), [q13] "v"(q[13]), [q14] "v"(q[14]), [q15] "v"(q[15]),
          [p0] "v"(p[0]), [p1] "v"(p[1]), [off] "v"(lane16), [src] "s"(c.src), [src2] "s"(c.src + 4096),
          [dst] "s"(c.dst)
        : "memory", "m0");
}

// The wait states after which vector ALU instructions may read what the last MFMAs wrote.
__device__ __forceinline__ void settle(floatx16 (&o)[8]) {
    asm volatile("s_nop 15\ns_nop 3\n"
                 : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]), "+v"(o[4]), "+v"(o[5]), "+v"(o[6]), "+v"(o[7]));
}
