#!/bin/bash
cd _work/exp2
for b in ringp ringp_noepi; do echo "== $b"
timeout -k 5 60 ./$b 2048 14336 4096 256 3 || exit 1
timeout -k 5 60 ./$b 2048 14336 4096 256 1 || exit 1
timeout -k 5 60 ./$b 2048 4096 4096 128 3 || exit 1
timeout -k 5 60 ./$b 2048 4096 4096 256 3 || exit 1
done
