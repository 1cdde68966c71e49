"""Writes tests/golden/http_contract.json: the control plane's contract as the reference's daemon
states it in its source TEXT (nothing of the reference is imported, compiled or run; its
third-party HTTP and JSON libraries are not in its tree). Read from
service/server/src/server.cpp (routes :28-39, handlers :204-543) and
service/common/src/convert.cpp (status fields :7-17):

  routes            [method, path] as registered
  status_fields     field name -> JSON type of an XQueue status object
  handlers          per handler function: the request keys and query parameters it reads, the
                    keys of the objects it answers with, and every (status code, literal body)
                    it can answer, in source order; a body of null is a bare status code

Run in the build container only:  python tests/golden/make_http_contract.py
tests/test_daemon_http.py checks the running daemon against the fixture."""
import json
import os
import re
import sys

REF = "/root/reference/service"
HERE = os.path.dirname(os.path.abspath(__file__))


def handlers_of(text):
    """name -> body text of every `... Server::Name(...) { ... }` definition."""
    out = {}
    for m in re.finditer(r"^[\w:<> ]+Server::(\w+)\([^)]*\)\s*\n\{", text, flags=re.M):
        depth, i = 1, m.end()
        while depth and i < len(text):
            depth += {"{": 1, "}": -1}.get(text[i], 0)
            i += 1
        out[m.group(1)] = text[m.end():i]
    return out


def answers_of(body):
    """(status, literal body or None) in source order: a status assignment applies to the next
    set_content or, when a return comes first, stands alone."""
    out, pending = [], None
    token = re.compile(r"res\.status\s*=\s*httplib::StatusCode::\w+_(\d+)|set_content\(\"((?:[^\"\\]|\\.)*)\"|\breturn\b")
    for m in token.finditer(body):
        if m.group(1):
            pending = int(m.group(1))
        elif m.group(2) is not None:
            literal = json.loads(m.group(2).replace('\\"', '"'))
            out.append([pending or 200, literal])
            pending = None
        else:
            if pending is not None:
                out.append([pending, None])
            pending = None
    uniq = []
    for a in out:
        if a not in uniq:
            uniq.append(a)
    return uniq


def main():
    server = open(os.path.join(REF, "server", "src", "server.cpp")).read()
    convert = open(os.path.join(REF, "common", "src", "convert.cpp")).read()
    contract = {"source": ["service/server/src/server.cpp", "service/common/src/convert.cpp"]}
    contract["routes"] = [[m.group(1).upper(), m.group(2)] for m in re.finditer(r'http_server_\.(Get|Post)\("([^"]+)"', server)]
    to_json = re.search(r"XQueueStatusToJson\(.*?\)\s*\{(.*?)\n\}", convert, flags=re.S).group(1)
    kinds = {"UInt64": "integer", "Int": "integer", "Int64": "integer"}
    contract["status_fields"] = {}
    for m in re.finditer(r'json\["(\w+)"\]\s*=\s*(?:\(Json::(\w+)\))?', to_json):
        contract["status_fields"][m.group(1)] = kinds.get(m.group(2), "boolean")
    contract["handlers"] = {}
    functions = handlers_of(server)
    for name, body in functions.items():
        if "httplib::Response" not in server[server.index("Server::" + name + "("):][:200]:
            continue
        # request keys read by the member functions a handler calls count as the handler's
        called = "".join(text for other, text in functions.items() if other != name and re.search(r"\b%s\(" % other, body))
        contract["handlers"][name] = {
            "request_keys": sorted(set(re.findall(r'request\["(\w+)"\]', body + called)) | set(re.findall(r'isMember\("(\w+)"\)', body + called))),
            "query_parameters": sorted(set(re.findall(r'has_param\("(\w+)"\)', body))),
            "path_parameters": sorted(set(re.findall(r'path_params\.at\("(\w+)"\)', body))),
            "response_keys": sorted(set(re.findall(r'response\["(\w+)"\]', body))),
            "process_keys": sorted(set(re.findall(r'process\["(\w+)"\]', body))),
            "answers": answers_of(body),
        }
    path = os.path.join(HERE, "http_contract.json")
    with open(path, "w") as f:
        json.dump(contract, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", path, "-", len(contract["routes"]), "routes,", len(contract["handlers"]), "handlers,",
          sum(len(h["answers"]) for h in contract["handlers"].values()), "answers")


if __name__ == "__main__":
    sys.exit(main())
