"""Writes tests/golden/abi_layout.json: sizeof/offsetof of the reference's structures.

Run in a container where the reference tree is mounted.  It compiles a few lines of
C that include the reference's own thnets.h where it lies (default build, and
-DLOWP) and prints the numbers; the JSON that results is the fixture the ABI tests
compare this repository's header and ctypes mirror against.

    python tests/golden/make_abi_layout.py [/root/reference]
"""
import json
import os
import subprocess
import sys
import tempfile

PROBE = r'''
#include <stdio.h>
#include <stddef.h>
#include "thnets.h"
#define S(name, type) printf("\"sizeof_%s\": %zu,\n", name, sizeof(type))
#define O(name, type, field) printf("\"off_%s\": %zu,\n", name, offsetof(type, field))
int main(void)
{
	printf("{\n");
	S("THFloatStorage", THFloatStorage);
	S("THFloatTensor", THFloatTensor);
	O("tensor_nDimension", THFloatTensor, nDimension);
	O("tensor_storage", THFloatTensor, storage);
	O("tensor_storageOffset", THFloatTensor, storageOffset);
	S("module", struct module);
	O("module_updateOutput", struct module, updateOutput);
	O("module_output", struct module, output);
	O("module_net", struct module, net);
	O("module_outputname", struct module, outputname);
	O("module_inputs", struct module, inputs);
	O("module_union", struct module, SpatialConvolution);
	S("SpatialConvolution", struct SpatialConvolution);
	O("conv_dW", struct SpatialConvolution, dW);
	O("conv_nOutputPlane", struct SpatialConvolution, nOutputPlane);
	S("SpatialFullConvolution", struct SpatialFullConvolution);
	O("fullconv_adjW", struct SpatialFullConvolution, adjW);
	O("fullconv_ones", struct SpatialFullConvolution, ones);
	S("SpatialMaxPooling", struct SpatialMaxPooling);
	O("maxpool_indices", struct SpatialMaxPooling, indices);
	S("SpatialBatchNormalization", struct SpatialBatchNormalization);
	O("bn_eps", struct SpatialBatchNormalization, eps);
	S("Linear", struct Linear);
	S("Threshold", struct Threshold);
	S("View", struct View);
	S("network", struct network);
	O("network_modules", struct network, modules);
	S("THNETWORK", THNETWORK);
	O("thnetwork_net", THNETWORK, net);
	O("thnetwork_out", THNETWORK, out);
	O("thnetwork_mean", THNETWORK, mean);
	O("thnetwork_std", THNETWORK, std);
	printf("\"n_module_types\": %d,\n", MT_Transpose + 1);
	printf("\"MT_Linear\": %d, \"MT_CAddTable\": %d, \"MT_SpatialBatchNormalization\": %d,\n",
		MT_Linear, MT_CAddTable, MT_SpatialBatchNormalization);
	printf("\"ENGINE_LOWP\": %d\n}\n", ENGINE_LOWP);
	return 0;
}
'''


def probe(ref, extra):
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "probe.c")
        exe = os.path.join(d, "probe")
        with open(src, "w") as f:
            f.write(PROBE)
        subprocess.check_call(["gcc", "-w", "-I", ref] + extra + ["-o", exe, src])
        return json.loads(subprocess.check_output([exe]).decode())


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = {"default": probe(ref, []), "lowp": probe(ref, ["-DLOWP"])}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "abi_layout.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote", path)


if __name__ == "__main__":
    main()
