    .section .rodata
    .balign 4096
psn_blob_0_begin:
    .incbin "/root/repo/openagents_amd/lib/psn_quant.gfx950.hsaco"
psn_blob_0_end:
    .balign 4096
psn_blob_1_begin:
    .incbin "/root/repo/openagents_amd/lib/psn_mv_q4_0.gfx950.hsaco"
psn_blob_1_end:
    .balign 4096
psn_blob_2_begin:
    .incbin "/root/repo/openagents_amd/lib/psn_mv_q8_0.gfx950.hsaco"
psn_blob_2_end:
    .balign 4096
psn_blob_3_begin:
    .incbin "/root/repo/openagents_amd/lib/psn_mv_q4_K.gfx950.hsaco"
psn_blob_3_end:
    .balign 4096
psn_blob_4_begin:
    .incbin "/root/repo/openagents_amd/lib/psn_mv_q6_K.gfx950.hsaco"
psn_blob_4_end:
    .balign 4096
psn_blob_5_begin:
    .incbin "/root/repo/openagents_amd/lib/psn_prefill.gfx950.hsaco"
psn_blob_5_end:
    .balign 4096
psn_blob_6_begin:
    .incbin "/root/repo/openagents_amd/lib/psn_decode.gfx950.hsaco"
psn_blob_6_end:
    .balign 16
    .globl psn_builtin_blobs
psn_builtin_blobs:
    .quad psn_blob_0_begin
    .quad psn_blob_0_end
    .quad psn_blob_1_begin
    .quad psn_blob_1_end
    .quad psn_blob_2_begin
    .quad psn_blob_2_end
    .quad psn_blob_3_begin
    .quad psn_blob_3_end
    .quad psn_blob_4_begin
    .quad psn_blob_4_end
    .quad psn_blob_5_begin
    .quad psn_blob_5_end
    .quad psn_blob_6_begin
    .quad psn_blob_6_end
    .balign 4
    .globl psn_builtin_blob_count
psn_builtin_blob_count:
    .long 7
    .section .note.GNU-stack,"",@progbits
