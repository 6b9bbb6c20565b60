/* The five kernel translation units compiled as bare gfx950 code objects
 * (reduce_*.hsaco, built by the Makefile), embedded read-only: the component
 * loads them through the HSA runtime for launches on its own dispatch queue.
 * Image i lies between xccl_rocm_kernel_image_begin[i] and ..._end[i]. */
    .section .rodata.xccl_rocm_images, "a", @progbits
    .balign 4096
img0: .incbin "reduce_w8.hsaco"
img0e:
    .balign 4096
img1: .incbin "reduce_w16.hsaco"
img1e:
    .balign 4096
img2: .incbin "reduce_w32.hsaco"
img2e:
    .balign 4096
img3: .incbin "reduce_w64.hsaco"
img3e:
    .balign 4096
img4: .incbin "reduce_fp.hsaco"
img4e:

    .section .data.rel.ro.xccl_rocm_images, "aw", @progbits
    .balign 8
    .globl xccl_rocm_kernel_image_begin
    .hidden xccl_rocm_kernel_image_begin
    .type xccl_rocm_kernel_image_begin, @object
xccl_rocm_kernel_image_begin:
    .quad img0, img1, img2, img3, img4
    .size xccl_rocm_kernel_image_begin, . - xccl_rocm_kernel_image_begin
    .globl xccl_rocm_kernel_image_end
    .hidden xccl_rocm_kernel_image_end
    .type xccl_rocm_kernel_image_end, @object
xccl_rocm_kernel_image_end:
    .quad img0e, img1e, img2e, img3e, img4e
    .size xccl_rocm_kernel_image_end, . - xccl_rocm_kernel_image_end
    .section .note.GNU-stack, "", @progbits
