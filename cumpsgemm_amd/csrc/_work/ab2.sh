#!/bin/bash
script=$1; shift
for rep in 1 2; do for v in "$@"; do timeout -k 10 200 python -u $script $v 2>&1 | grep -v amdgpu.ids || exit 1; done; done
