"""Writes tests/golden/train_profile_reference.csv: the header and the first two epochs (138 rows) of the one
event log the reference holds, /root/reference/train-profile.csv (dataset 1000, global batch 500, micro-batch
32: every global batch is 15 micro-batches of 32 and one of 20; one optimizer step per global batch).  The
rows are data the reference's own run wrote; nothing else of the reference is read.  Run in the build
container (the reference is not on the GPU box):

    python tests/golden/make_profile_fixture.py
"""
import os

SRC = "/root/reference/train-profile.csv"
DST = os.path.join(os.path.dirname(os.path.abspath(__file__)), "train_profile_reference.csv")


def main():
    with open(SRC) as f:
        lines = f.read().splitlines()
    out = [lines[0]]
    for line in lines[1:]:
        name = line.split(",")[1] if "," in line else ""
        if name.startswith("epoch_02_"):
            break
        out.append(line)
    with open(DST, "w") as f:
        f.write("\n".join(out) + "\n")
    print(f"{DST}: {len(out) - 1} rows")


if __name__ == "__main__":
    main()
