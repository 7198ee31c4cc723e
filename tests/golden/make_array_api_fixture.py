"""Writes tests/golden/array_api_clusters.json from the reference's graph dumps.

Input: docs/array_api_values.svg and docs/array_api_grad.svg of the reference repository -- graphviz renderings
of `Graph::write_dot(KernelDotOutput::Cluster)` (src/graph.rs:661-763) for the two graphs of
examples/array_api/main.rs.  The files are read as text (they are drawings, not code); nodes are assigned to
clusters by geometric containment of the node's first label inside a cluster rectangle.

Output: for each graph, the list of clusters as sorted op labels, the labels outside any cluster (inputs,
outputs, inlined literals), and the edges between labelled nodes.

Run in the build container only:  python tests/golden/make_array_api_fixture.py /root/reference
"""
import json
import os
import re
import sys


def parse(svg_text):
    clusters = []
    for m in re.finditer(r'<g\s+id="clust\d+"\s+class="cluster">(.*?)</g>', svg_text, re.S):
        pts = re.search(r'points="([^"]+)"', m.group(1)).group(1).split()
        xs = [float(p.split(",")[0]) for p in pts]
        ys = [float(p.split(",")[1]) for p in pts]
        clusters.append((min(xs), max(xs), min(ys), max(ys)))
    nodes = {}
    for m in re.finditer(r'<g\s+id="node\d+"\s+class="node">(.*?)</g>', svg_text, re.S):
        body = m.group(1)
        name = re.search(r"<title[^>]*>([^<]+)</title>", body).group(1)
        texts = re.findall(r'<text[^>]*?x="([-\d.]+)"\s+y="([-\d.]+)"[^>]*>([^<]*)</text>', body, re.S)
        x, y, label = float(texts[0][0]), float(texts[0][1]), texts[0][2]
        shape = texts[1][2] if len(texts) > 1 else ""
        inside = [i for i, (x0, x1, y0, y1) in enumerate(clusters) if x0 <= x <= x1 and y0 <= y <= y1]
        nodes[name] = {"label": label, "shape": shape, "cluster": inside[0] if inside else None}
    edges = []
    for m in re.finditer(r'<g\s+id="edge\d+"\s+class="edge">(.*?)</g>', svg_text, re.S):
        t = re.search(r"<title[^>]*>([^<]+)</title>", m.group(1)).group(1)
        a, b = t.replace("&#45;", "-").replace("&gt;", ">").split("->")
        edges.append([nodes[a]["label"], nodes[b]["label"]])
    out_clusters = []
    for i in range(len(clusters)):
        out_clusters.append(sorted(n["label"] for n in nodes.values() if n["cluster"] == i))
    outside = sorted(n["label"] for n in nodes.values() if n["cluster"] is None)
    return {"clusters": sorted(out_clusters), "outside": outside, "edges": sorted(edges)}


if __name__ == "__main__":
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = {}
    for key, name in (("values", "array_api_values.svg"), ("grad", "array_api_grad.svg")):
        out[key] = parse(open(os.path.join(ref, "docs", name)).read())
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "array_api_clusters.json")
    json.dump(out, open(path, "w"), indent=1)
    print(json.dumps(out, indent=1))
