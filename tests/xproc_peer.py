"""One side of the two-process transfer test (tests/test_cross_process.py starts this file
twice as child programs, a target and an initiator, on the same GPU).

target:    registers 8 MiB of VRAM (first half zero, second half a known pattern), writes its
           metadata blob to <dir>/target.md, waits for the initiator's notification, checks
           that its first half now holds the initiator's pattern, waits for "bye".
initiator: loads the blob, WRITEs its pattern into the target's first half with a
           notification attached, READs the target's second half and checks it, says "bye".
Shape of the reference's two-agent test, test/unit/plugins/ucx/ucx_backend_test.cpp (separate
engines, metadata exchanged as blobs, byte compare after READ and WRITE).
"""
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import numpy as np  # noqa: E402
import torch  # noqa: E402

from nixl_amd import nixl_agent, nixl_agent_config  # noqa: E402

HALF = 4 << 20


def pattern(seed, n=HALF):
    return torch.from_numpy(np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8))


def wait_for(cond, what, seconds=90.0):
    t0 = time.time()
    while time.time() - t0 < seconds:
        v = cond()
        if v:
            return v
        time.sleep(0.005)
    raise SystemExit(f"timed out waiting for {what}")


def target(workdir):
    dev = torch.device("cuda:0")
    buf = torch.zeros(2 * HALF, dtype=torch.uint8, device=dev)
    buf[HALF:] = pattern(7).to(dev)
    torch.cuda.synchronize()
    agent = nixl_agent("T", nixl_agent_config(backends=("HIP",)))
    agent.register_memory([buf])
    with open(os.path.join(workdir, "target.addr"), "w") as f:
        f.write(str(buf.data_ptr()))
    tmp = os.path.join(workdir, "target.md.tmp")
    with open(tmp, "wb") as f:
        f.write(agent.get_agent_metadata())
    os.rename(tmp, os.path.join(workdir, "target.md"))
    got = {}

    def notified(tag):
        agent.update_notifs()
        return any(m == tag for m in agent.notifs.get("I", []))

    wait_for(lambda: notified(b"written"), "the initiator's notification")
    torch.cuda.synchronize()
    if not torch.equal(buf[:HALF].cpu(), pattern(11)):
        raise SystemExit("target: the bytes the initiator wrote are wrong")
    if not torch.equal(buf[HALF:].cpu(), pattern(7)):
        raise SystemExit("target: bytes outside the written range changed")
    wait_for(lambda: notified(b"bye"), "the initiator's goodbye")
    agent.close()
    print("target OK", flush=True)


def initiator(workdir):
    dev = torch.device("cuda:0")
    md_path = os.path.join(workdir, "target.md")
    wait_for(lambda: os.path.exists(md_path), "the target's metadata")
    local = torch.zeros(2 * HALF, dtype=torch.uint8, device=dev)
    local[:HALF] = pattern(11).to(dev)
    torch.cuda.synchronize()
    agent = nixl_agent("I", nixl_agent_config(backends=("HIP",)))
    agent.register_memory([local])
    with open(md_path, "rb") as f:
        blob = f.read()
    with open(os.path.join(workdir, "target.addr")) as f:
        remote_base = int(f.read())
    # A blob that claims a region (and an allocation) far longer than what the target shares is
    # refused when it is loaded: the region is checked against the mapping as seen here.
    import struct
    honest = struct.pack("<QQ", remote_base, 2 * HALF)
    at = blob.find(b"HIPREGN2")
    if at < 0 or blob.count(honest) < 2:
        raise SystemExit("initiator: the metadata blob does not look as expected")
    forged = bytearray(blob.replace(honest, struct.pack("<QQ", remote_base, 1 << 30)))
    forged[at + 48:at + 56] = struct.pack("<Q", (1 << 30) + (512 << 20))  # alloc_size
    try:
        agent.add_remote_agent(bytes(forged))
    except Exception as e:
        print("initiator: forged blob refused:", e, flush=True)
    else:
        raise SystemExit("initiator: a region longer than the target's allocation was accepted")
    name = agent.add_remote_agent(blob)
    assert name == "T", name
    triple = lambda a: np.array([[a, HALF, 0]], dtype=np.uint64)
    # WRITE local first half -> target first half, with a notification that must not overtake the bytes
    w = agent.initialize_xfer("WRITE", agent.get_xfer_descs(triple(local.data_ptr()), "VRAM"),
                              agent.get_xfer_descs(triple(remote_base), "VRAM"), "T", notif_msg=b"written")
    state = agent.transfer(w)
    while state == "PROC":
        state = agent.check_xfer_state(w)
    assert state == "DONE", state
    # READ target second half -> local second half
    r = agent.initialize_xfer("READ", agent.get_xfer_descs(triple(local.data_ptr() + HALF), "VRAM"),
                              agent.get_xfer_descs(triple(remote_base + HALF), "VRAM"), "T")
    state = agent.transfer(r)
    while state == "PROC":
        state = agent.check_xfer_state(r)
    assert state == "DONE", state
    torch.cuda.synchronize()
    if not torch.equal(local[HALF:].cpu(), pattern(7)):
        raise SystemExit("initiator: the bytes read from the target are wrong")
    # a range that sticks out of the target's registration is refused on the host
    try:
        agent.initialize_xfer("WRITE", agent.get_xfer_descs(triple(local.data_ptr()), "VRAM"),
                              agent.get_xfer_descs(triple(remote_base + HALF + 4096), "VRAM"), "T")
    except Exception:
        pass
    else:
        raise SystemExit("initiator: a transfer beyond the target's region was accepted")
    agent.send_notif("T", b"bye")
    w.release()
    r.release()
    agent.remove_remote_agent("T")
    agent.close()
    print("initiator OK", flush=True)


if __name__ == "__main__":
    {"target": target, "initiator": initiator}[sys.argv[1]](sys.argv[2])
