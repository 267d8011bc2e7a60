#!/bin/bash
# VGG-16 conv layers, one driver invocation per distinct layer shape (the layer
# list of the reference's run_vgg16.sh).
# usage: ./run_vgg16.sh -a <auto|winograd|im2col> -tn <no_tuning|tuning> -i <iterations> [-n <batch> [driver options]]
algo=$2
tuning=$4
iterations=$6
batch=${8:-1}
extra="${@:9}"      # anything after the batch goes to the driver as it is (--check-images 1, --no-check, --strict)
BIN="$(dirname "$0")/../bin/conv_test"

for layer in "3 64 224" "64 64 224" "64 128 112" "128 128 112" "128 256 56" "256 256 56" "256 512 28" "512 512 28" "512 512 14"; do
    set -- $layer
    $BIN -ic $1 -oc $2 -is $3 $3 -ks 3 3 -ip 1 -a $algo -tn $tuning -i $iterations -n $batch -t 16 --json $extra || exit 1
done
