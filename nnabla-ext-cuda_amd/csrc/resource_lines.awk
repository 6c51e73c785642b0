# Folds the compiler's kernel-resource-usage remarks into one line per kernel:
#   <mangled name> sgpr=<n> vgpr=<n> agpr=<n> scratch=<bytes/lane> lds=<bytes/block> occupancy=<waves/SIMD>
/remark: Function Name:/ { if (name != "") emit(); name = $0; sub(/.*Function Name: /, "", name); sub(/ \[-Rpass.*/, "", name) }
/remark: +TotalSGPRs:/ { sgpr = field($0) }
/remark: +VGPRs:/ { vgpr = field($0) }
/remark: +AGPRs:/ { agpr = field($0) }
/remark: +ScratchSize/ { scratch = field($0) }
/remark: +Occupancy/ { occ = field($0) }
/remark: +LDS Size/ { lds = field($0) }
END { if (name != "") emit() }
function field(line) { sub(/ \[-Rpass.*/, "", line); sub(/.*: /, "", line); return line }
function emit() { print name, "sgpr=" sgpr, "vgpr=" vgpr, "agpr=" agpr, "scratch=" scratch, "lds=" lds, "occupancy=" occ }
