/* Embeds the gfx950 code objects in the runtime library's read-only data, one
 * begin/end symbol pair per module.  The assembler resolves the file names
 * against the include path (-I <build dir>). */
        .section .rodata.hcamd_blobs, "a", @progbits

        .macro hcamd_blob name
        .balign 4096
        .global hcamd_blob_\name\()_begin
        .type hcamd_blob_\name\()_begin, @object
hcamd_blob_\name\()_begin:
        .incbin "\name\().hsaco"
        .global hcamd_blob_\name\()_end
        .type hcamd_blob_\name\()_end, @object
hcamd_blob_\name\()_end:
        .byte 0
        .endm

        hcamd_blob copy
        hcamd_blob elementwise
        hcamd_blob map
        hcamd_blob imap
        hcamd_blob fmap
        hcamd_blob distance
        hcamd_blob gather
        hcamd_blob softmax
        hcamd_blob quantize
        hcamd_blob gemm

        .section .note.GNU-stack, "", @progbits
