from .build import build_all

if __name__ == "__main__":
    build_all()
