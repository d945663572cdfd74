"""Energy server: JSON requests for the energy and gradient of one molecule.

Wire format of the reference's energy_server.py:141-187 over the naive socket protocol of
client_server.py:8-41 (one UTF-8 JSON document per send, at most 1 MiB per receive):

    request   {"X": [[type, x, y, z], ...]}          type 0=H 1=C 2=N 3=O, coordinates in Angstrom
    response  {"energy": E, "gradient": [g0x, g0y, g0z, g1x, ...]}

E is the network's energy plus the atoms' self-interaction energies (Hartree); the gradient is d E / d xyz
converted from Hartree/Angstrom to Hartree/Bohr by multiplying with 0.52917721092, as the reference does
(energy_server.py:179-181).
"""
import json
import socket

import numpy as np

from .batching import RawDataset

BOHR = 0.52917721092          # energy_server.py:18
ENCODING = "utf-8"            # client_server.py:4
MAX_BYTES = 1024 ** 2         # client_server.py:5
BACKLOG = 10                  # client_server.py:6

# wB97X/6-31G(d) self-interaction energies of H, C, N, O in Hartree (data_utils.py:28-33, stored as float32 there)
SELF_INTERACTION = np.array([-0.49932123901, -37.83271996200, -54.57325122225, -75.04147134502], dtype=np.float32)


def parse_request(text):
    """JSON text -> float64 array [n_atoms, 4] of (type, x, y, z) rows (energy_server.py:152-154)."""
    doc = json.loads(text)
    X = doc.get("X") if isinstance(doc, dict) else None
    if X is None:
        raise ValueError('the request has no "X"')
    X_np = np.array(X, dtype=np.float64)
    if X_np.ndim != 2 or X_np.shape[1] != 4 or X_np.shape[0] == 0:
        raise ValueError('"X" must be a non-empty list of [type, x, y, z] rows')
    types = X_np[:, 0]
    if np.any(types != np.round(types)) or np.any(types < 0) or np.any(types > 3):
        raise ValueError("atom types must be 0 (H), 1 (C), 2 (N) or 3 (O)")
    return X_np


def self_interaction(X_np):
    """Sum of the atoms' self-interaction energies (energy_server.py:159-162)."""
    return float(sum(SELF_INTERACTION[int(row[0])] for row in X_np))


def format_response(energy, gradient):
    """energy in Hartree, gradient [n_atoms, 3] in Hartree/Angstrom -> JSON text (energy_server.py:164-185)."""
    flat = np.asarray(gradient, dtype=np.float64).reshape(-1)
    return json.dumps({"energy": float(energy), "gradient": [float(g) * BOHR for g in flat]})


def handle_request(model, text):
    """One request through `model` (an AniModel): -> response text."""
    X_np = parse_request(text)
    rd = RawDataset([X_np], [0.0])
    energy = float(model.predict(rd)[0]) + self_interaction(X_np)
    gradient = list(model.coordinate_gradients(rd))[0]
    return format_response(energy, gradient)


# ---------------------------------------------------------------------------- sockets (client_server.py:8-41)
def connect_socket(host, port, server=True):
    s = socket.socket(socket.AF_INET, socket.SOCK_STREAM)
    if server:
        s.setsockopt(socket.SOL_SOCKET, socket.SO_REUSEADDR, 1)
        s.bind((host, port))
        s.listen(BACKLOG)
    else:
        s.connect((socket.gethostbyname(host), port))
    return s


def send(s, data):
    s.sendall(bytes(data, encoding=ENCODING))


def receive(s):
    return s.recv(MAX_BYTES).decode(ENCODING)


recieve = receive          # the reference's spelling (client_server.py:32)


def close_connection(s):
    s.close()


def receive_request(conn, idle_s=0.25):
    """One JSON request from a connection that has no framing (the reference reads a single recv of up to 1 MB,
    client_server.py:29-34, which cuts a request that arrives in several segments): reads until the text parses
    as JSON, the peer closes, MAX_BYTES are in, or nothing more arrives for `idle_s` seconds after a partial
    message.  Returns the text ('' when the peer closed without sending); bytes that are not valid UTF-8 come
    back as a text that does not parse, so the caller answers with an error instead of dying."""
    buf = b""
    conn.settimeout(None)
    try:
        while len(buf) < MAX_BYTES:
            try:
                chunk = conn.recv(MAX_BYTES - len(buf))
            except socket.timeout:
                break
            if not chunk:
                break
            buf += chunk
            try:
                json.loads(buf.decode(ENCODING))
                break                                   # a complete request
            except (UnicodeDecodeError, ValueError):
                conn.settimeout(idle_s)                 # wait a little for the rest
    finally:
        conn.settimeout(None)
    return buf.decode(ENCODING, errors="replace")


def serve_on(s, model, max_connections=None):
    """Accepts connections on the listening socket `s` one at a time and answers requests until the peer closes
    (energy_server.py:137-190).  `max_connections` ends the loop after that many connections (None: forever).
    Closes `s` on the way out."""
    served = 0
    try:
        while max_connections is None or served < max_connections:
            conn, _ = s.accept()
            try:
                while True:
                    text = receive_request(conn)
                    if not text:
                        break
                    try:
                        reply = handle_request(model, text)
                    except (ValueError, KeyError, TypeError, IndexError) as e:   # malformed request: say so, keep serving
                        reply = json.dumps({"error": str(e)})
                    send(conn, reply)
            except OSError:
                pass                                            # the peer went away mid-request: next connection
            finally:
                conn.close()
            served += 1
    finally:
        s.close()


def serve(model, host, port, max_connections=None):
    serve_on(connect_socket(host, port, server=True), model, max_connections)


def main(argv=None):
    import argparse
    import os

    import torch

    from . import model as khan_model
    ap = argparse.ArgumentParser(description="server for energy requests")
    ap.add_argument("--save-dir", default="~/work", help="directory holding save_file.npz")
    ap.add_argument("--host", default="127.0.0.1")
    ap.add_argument("--port", default=5000, type=int)
    ap.add_argument("--deep-network", action="store_true")
    ap.add_argument("--fit-charges", action="store_true")
    ap.add_argument("--activation-function", default="celu", choices=sorted(khan_model.ACTIVATIONS))
    args = ap.parse_args(argv)
    save_file = os.path.join(os.path.expanduser(args.save_dir), "save_file.npz")
    if not os.path.exists(save_file):
        raise IOError("Saved NN numpy file does not exist")
    layers = khan_model.DEEP_LAYERS if args.deep_network else khan_model.DEFAULT_LAYERS
    m = khan_model.AniModel(layers, khan_model.get_fn_by_name(args.activation_function), torch.float64, "cuda:0",
                            fit_charges=args.fit_charges)
    m.load_numpy(save_file, strict=False)
    serve(m, args.host, args.port)


if __name__ == "__main__":
    main()
