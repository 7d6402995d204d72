"""Writes tests/golden/otter_syntax_cases.dump: what the COMPILED REFERENCE's parser (Tensor/Otter.cpp, through
oracle/_ref/libotter_ref.so) makes of tests/golden/otter_syntax_cases.otter. Run here, where /root/reference exists:

    make -C oracle ref && python tests/golden/make_model_file_fixtures.py

tests/golden/nanodet-plus-m-1.5x_416_int8_fused.otter is a data file of the reference (benchmark/, the description of
its int8 detection model; it ships no weights), kept here because the GPU box has no copy of the reference."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.binding import Ref  # noqa: E402

if __name__ == "__main__":
    dump = Ref().otter_dump(os.path.join(HERE, "otter_syntax_cases.otter"))
    with open(os.path.join(HERE, "otter_syntax_cases.dump"), "w") as f:
        f.write(dump)
    print("wrote %d lines" % len(dump.splitlines()))
