#!/bin/sh
# oracle/_ref: a checker built from the reference's own sources.
#
# Not buildable in this image: the CPU functions of the path (finchmoe/infer.m:690-702,
# 1575-1881) live inside infer.m, a 15,958-line Objective-C unit that needs Foundation,
# Metal, Accelerate and GCD headers (infer.m:45-69); there is no Objective-C runtime, no
# Apple SDK and no way to compile that file directly, and no stand-in headers are written.
# The reference's Python format tools are read, not run.  So nothing is produced here and
# the oracle is pinned by the checks listed in fm_oracle.h.
if [ -d /root/reference/finchmoe ]; then
    echo "oracle/_ref: reference path lives in infer.m (needs Foundation/Metal): unbuildable here, skipped"
fi
exit 0
