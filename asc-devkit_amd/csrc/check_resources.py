"""Collects the per-kernel resource figures that hipcc prints with -Rpass-analysis=kernel-resource-usage.

usage: check_resources.py a.remarks b.remarks ...   (JSON on stdout, exit status 1 when a guarded kernel has scratch)

A guarded kernel reads LDS or global memory through inline assembly (`ds_read_b128`, `global_load_lds`) and makes the
result visible to the compiler only at a later counted wait.  Until then the compiler takes the destination registers
for valid.  If register pressure makes it spill or copy one of them in between, stale data is stored, or the load that
is still in flight writes into a register that now belongs to something else (a memory fault was seen from exactly
this).  A scratch frame of zero bytes and zero spilled vector registers is the build-time proof that no such move
exists.  Spilled scalar registers are recorded but allowed: the compiler parks them in lanes of a vector register it
reserves for that purpose, which is never the destination of a load.
"""
import json
import re
import subprocess
import sys

# kernels built on the inline-assembly read pattern, by the name they have in the sources
GUARDED = ("gemm_nkl_kernel", "w8a16_nk_stream_kernel", "w4a16_gemv_kernel", "w4a16_tile_kernel", "w8a16_tile_kernel", "gemm_stream_kernel", "gemm_dma_kernel",
           "gemm_dma_dual_kernel", "gemm_dma_group_kernel", "w4a16_packed_kernel", "w4a16_packed_rows_kernel",
           "gemm_packed_kernel", "gemm_packed_dyn_kernel", "gemm_ws_kernel", "mx_tile_kernel")

FIELDS = {
    "TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes_per_lane",
    "Occupancy [waves/SIMD]": "waves_per_simd", "SGPRs Spill": "sgpr_spills", "VGPRs Spill": "vgpr_spills",
    "LDS Size [bytes/block]": "lds_bytes",
}


def demangle(names):
    out = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True, check=True).stdout
    return out.splitlines()


def parse(path):
    kernels, cur = [], None
    for line in open(path, errors="replace"):
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            cur = {"symbol": m.group(1), "file": path.rsplit("/", 1)[-1].replace(".remarks", ".hip")}
            kernels.append(cur)
            continue
        m = re.search(r"remark:\s+([A-Za-z \[\]/]+): (\d+)", line)
        if m and cur is not None and m.group(1).strip() in FIELDS:
            cur[FIELDS[m.group(1).strip()]] = int(m.group(2))
    return kernels


def main(paths):
    kernels = [k for p in paths for k in parse(p)]
    if not kernels:
        sys.stderr.write("check_resources: no kernel remarks found in %s\n" % " ".join(paths))
        return 1
    for k, name in zip(kernels, demangle([k["symbol"] for k in kernels])):
        k["name"] = name.replace("ascq::(anonymous namespace)::", "")
        base = re.sub(r"^void ", "", k["name"]).split("<")[0].split("(")[0]
        k["guarded"] = base in GUARDED
    bad = [k for k in kernels if k["guarded"] and (k.get("scratch_bytes_per_lane", 1) or k.get("vgpr_spills", 1))]
    json.dump({"guarded_names": GUARDED, "kernels": kernels}, sys.stdout, indent=1)
    for k in bad:
        sys.stderr.write("check_resources: %s (%s) has %d bytes of scratch per lane, %d VGPR and %d SGPR spills; a kernel "
                         "with inline-assembly loads must have none\n" % (k["name"], k["file"], k.get(
                             "scratch_bytes_per_lane", -1), k.get("vgpr_spills", -1), k.get("sgpr_spills", -1)))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
