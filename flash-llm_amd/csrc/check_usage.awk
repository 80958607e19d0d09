# Reads the compiler's kernel-resource-usage remarks of one object file and fails (exit 1) when a kernel that the
# launch code's assumptions depend on came out differently:
#   spmm_stream_kernel  every instance must keep two waves per SIMD (the grids are sized for eight waves per CU);
#   spmm_group_kernel   issues its MFMAs as inline assembly on accumulators that must stay where they are: the
#                       build that was verified has 168 VGPRs or fewer and three waves per SIMD (launch bounds);
#                       more registers or a lower occupancy means the compiler started moving accumulators.
/Function Name:/ { name = $0 }
/ VGPRs: /       { split($0, a, "VGPRs: "); vgprs = a[2] + 0 }
/Occupancy \[waves\/SIMD\]:/ {
    split($0, a, "SIMD]: "); occ = a[2] + 0
    if (name ~ /spmm_stream_kernel/ && occ < 2) { print "spmm_stream_kernel: occupancy " occ " < 2: " name; bad = 1 }
    if (name ~ /spmm_group_kernel/ && (occ < 3 || vgprs > 168)) { print "spmm_group_kernel: " vgprs " VGPRs, occupancy " occ ": " name; bad = 1 }
}
END { exit bad }
