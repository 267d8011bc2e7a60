#!/bin/bash
# ResNet-50 conv layers (the layer list of the reference's run_resnet50.sh, which puts
# stride 2 on the 1x1 projections), plus the 3x3 stride-2 layers of the v1.5 variant.
# usage: ./run_resnet50.sh -a <auto|winograd|im2col> -tn <no_tuning|tuning> -i <iterations> [-n <batch> [driver options]]
algo=$2
tuning=$4
iterations=$6
batch=${8:-1}
extra="${@:9}"      # anything after the batch goes to the driver as it is (--check-images 1, --no-check, --strict)
BIN="$(dirname "$0")/../bin/conv_test"
run() { $BIN "$@" -a $algo -tn $tuning -i $iterations -n $batch -t 16 --json $extra || exit 1; }

run -ic 3    -oc 64   -is 224 224 -ks 7 7 -ip 3 -s 2 2
run -ic 64   -oc 64   -is 56 56   -ks 1 1 -ip 0 -s 1 1
run -ic 64   -oc 64   -is 56 56   -ks 3 3 -ip 1 -s 1 1
run -ic 64   -oc 256  -is 56 56   -ks 1 1 -ip 0 -s 1 1
run -ic 256  -oc 64   -is 56 56   -ks 1 1 -ip 0 -s 1 1
run -ic 256  -oc 128  -is 56 56   -ks 1 1 -ip 0 -s 2 2
run -ic 128  -oc 128  -is 28 28   -ks 3 3 -ip 1 -s 1 1
run -ic 128  -oc 512  -is 28 28   -ks 1 1 -ip 0 -s 1 1
run -ic 256  -oc 512  -is 56 56   -ks 1 1 -ip 0 -s 2 2
run -ic 512  -oc 128  -is 28 28   -ks 1 1 -ip 0 -s 1 1
run -ic 512  -oc 256  -is 28 28   -ks 1 1 -ip 0 -s 2 2
run -ic 256  -oc 256  -is 14 14   -ks 3 3 -ip 1 -s 1 1
run -ic 256  -oc 1024 -is 14 14   -ks 1 1 -ip 0 -s 1 1
run -ic 512  -oc 1024 -is 28 28   -ks 1 1 -ip 0 -s 2 2
run -ic 1024 -oc 256  -is 14 14   -ks 1 1 -ip 0 -s 1 1
run -ic 1024 -oc 512  -is 14 14   -ks 1 1 -ip 0 -s 2 2
run -ic 512  -oc 512  -is 7 7     -ks 3 3 -ip 1 -s 1 1
run -ic 512  -oc 2048 -is 7 7     -ks 1 1 -ip 0 -s 1 1
run -ic 1024 -oc 2048 -is 14 14   -ks 1 1 -ip 0 -s 2 2
run -ic 2048 -oc 512  -is 7 7     -ks 1 1 -ip 0 -s 1 1
# 3x3 stride-2 layers (v1.5 placement of the stride)
run -ic 128  -oc 128  -is 56 56   -ks 3 3 -ip 1 -s 2 2
run -ic 256  -oc 256  -is 28 28   -ks 3 3 -ip 1 -s 2 2
run -ic 512  -oc 512  -is 14 14   -ks 3 3 -ip 1 -s 2 2
