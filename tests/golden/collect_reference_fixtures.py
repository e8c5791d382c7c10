"""Copies the data fixtures the reference's own tests hold for the fingerprint path
into tests/golden/ (run once in the authoring container; /root/reference is not
available on the GPU box).  Only data files are taken: a frame, exported model
parameters (text .dat, .npz weights), cutoff curves and recorded known answers.

  python tests/golden/collect_reference_fixtures.py [/root/reference]
"""
import json
import os
import shutil
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def cp(src, dst):
    os.makedirs(os.path.dirname(os.path.join(HERE, dst)), exist_ok=True)
    shutil.copyfile(os.path.join(REF, src), os.path.join(HERE, dst))
    os.chmod(os.path.join(HERE, dst), 0o644)


# F1: real 768-atom MB-pol water frame
for f in ("pos_0", "box_0", "type.dat"):
    cp(f"test/test-inference-pipeline/frames/{f}", f"frame_mbpol/{f}")
# F2: jittered copy in LAMMPS data format
cp("test/test-lammps-smoke/data.water_smoke", "frame_mbpol/data.water_smoke")
# F3: trained model, same checkpoint in fp32 and fp64 (parameters + MLP weights)
for prec, d in (("float", "model_onnx_grad_float"), ("double", "model_onnx_double")):
    for k in (0, 1):
        for f in ("alpha_2body", "alpha_3body", "type_emb_2b", "type_emb_3b", "type_emb_2b_sq", "type_emb_3b_sq",
                  "alpha_mu"):
            cp(f"test/test-lammps-smoke/{d}/type{k}_{f}.dat", f"model_{prec}/type{k}_{f}.dat")
        cp(f"test/test-lammps-smoke/{d}/mlp_type{k}.npz", f"model_{prec}/mlp_type{k}.npz")
        cp(f"test/test-lammps-smoke/{d}/mlp_type{k}.bin", f"model_{prec}/mlp_type{k}.bin")
    cp(f"test/test-lammps-smoke/{d}/type.dat", f"model_{prec}/type.dat")
    cp(f"test/test-lammps-smoke/{d}/staf_jmd.cfg", f"model_{prec}/staf_jmd.cfg")
cp("test/test-lammps-STAF-inference-STAF-comp/model_tf_float_log0/cutoff_info", "model_float/cutoff_info")
cp("test/test-lammps-STAF-inference-STAF-comp/model_tf_float_log0/cutoff_info", "model_double/cutoff_info")
# F5: cutoff curves written by fill_repulsion (fp32 and fp64 builds)
cp("test/test-inference-pipeline/cutoff_curve.dat", "cutoff_curve_float.dat")
cp("test/test-lammps-smoke/model_onnx_double/cutoff_curve.dat", "cutoff_curve_double.dat")
# F8: single-species example (nt = 1 shapes)
for f in ("pos_0", "box_0"):
    cp(f"STAF/example_inference/{f}", f"frame_single_species/{f}")
for f in ("cutoff_info", "type.dat", "type0_alpha_2body.dat", "type0_alpha_3body.dat"):
    cp(f"STAF/example_inference/model29/{f}", f"frame_single_species/{f}")
# F4/F6/F7: known answers recorded by the reference's own test runs
known = {
    "source": {
        "E_python/E_lammps/rms_F": "test/test-lammps-STAF-inference-STAF-comp/results/frames.csv:2",
        "PE_water_smoke": "test/B_ARCHITECTURE.md:167",
        "neighbours": "README.md:38",
        "intmap_counts": "test/test-inference-pipeline/comparison_summary.txt:32-33",
        "fill_repulsion_fp64": "closed form of STAF/src/descriptor_builder/reforce.cc:101-141 at Rc=4.5, Rs=2.25",
    },
    "frame0_model_float": {"E_python": -102.25880432128906, "E_lammps": -102.25872,
                           "rms_F_python": 0.6993059698907058, "max_abs_dF_python_vs_lammps": 4.42397937774619e-05},
    "water_smoke_model_float": {"PE": -99.53378},
    "mean_neighbours": 38.2, "mean_neighbours_sigma": 0.8,
    "intmap2b_elems_10_frames": 468480, "intmap3b_elems_10_frames": 27187200,
}
with open(os.path.join(HERE, "known_answers.json"), "w") as f:
    json.dump(known, f, indent=1)
print("fixtures written under", HERE)
