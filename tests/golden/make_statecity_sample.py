"""Writes tests/golden/statecity_sample.csv from the reference's demo data file
(demo/statecity.csv: US places with state, FIPS codes, name, type, latitude,
longitude; 29,510 rows).  Kept: the rows of a dozen states, large and small,
in file order (the file is sorted by state), with the three columns the
nearest-cities pipeline of demo/cities.cu reads: state, latitude, longitude.

    python tests/golden/make_statecity_sample.py /root/reference/demo/statecity.csv
"""
import csv
import os
import sys

STATES = ["AK", "AZ", "CT", "DC", "DE", "HI", "MA", "NV", "RI", "UT", "VT", "WY"]


def main(source):
    here = os.path.dirname(os.path.abspath(__file__))
    rows = []
    with open(source, newline="") as f:
        reader = csv.reader(f)
        next(reader)
        for row in reader:
            if row[0] in STATES:
                rows.append((row[0], row[-2].strip(), row[-1].strip()))
    with open(os.path.join(here, "statecity_sample.csv"), "w") as f:
        f.write("state,latitude,longitude\n")
        for state, lat, lon in rows:
            f.write("%s,%s,%s\n" % (state, lat, lon))
    print(len(rows), "rows")


if __name__ == "__main__":
    main(sys.argv[1])
