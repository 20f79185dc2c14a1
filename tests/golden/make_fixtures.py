"""Regenerates the JSON fixtures of this folder from the transcription scripts beside it.

    python tests/golden/make_fixtures.py        (from the repository root)

Every script holds known-answer vectors typed in by hand from the reference's own #[test]s (each case names its file:lines
under libs/rtensors/src/); none of them reads or runs the reference.  The three view scripts append to one file and must run in
order.  reference_reduce_stat_vectors.json was written by hand and has no script."""
import os
import runpy

HERE = os.path.dirname(os.path.abspath(__file__))
ORDER = ["make_reference_vectors.py", "make_reference_scalar_vectors.py", "make_reference_view_vectors_1.py",
         "make_reference_view_vectors_2.py", "make_reference_view_vectors_3.py", "make_reference_operand_vectors.py",
         "make_reference_matmul_vectors.py"]

if __name__ == "__main__":
    os.chdir(os.path.dirname(os.path.dirname(HERE)))
    for name in ORDER:
        runpy.run_path(os.path.join(HERE, name), run_name="__main__")
